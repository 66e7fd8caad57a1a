// RMS norm in groups, around a sublayer: the result y of a mixer or feed-forward is normed, added to the 32-bit
// residual stream, and the sum is normed again for the sublayer that follows, in one kernel.
//
//   norm_g(v)[c] = w[c] * v[c] / sqrt(mean(v[group of c]^2) + eps)     the row cut into `groups` equal consecutive parts
//
//   resid[r] += norm_g(y[r]; post_w)     (post_w == nullptr: y is added as it is; y == nullptr: nothing is added)
//   out[r]    = norm_g(resid[r]; pre_w)  (out == nullptr: no second norm; pre_w == nullptr: out[r] = resid[r], rounded,
//                                         for a sublayer that reads the residual stream as it is)
//
// rows == nullptr: every row, the residual updated in place. rows != nullptr: row rows[r] is read, nothing is written
// back, out row r (the rows whose logits are wanted).
//
// Everything is 32-bit; a bfloat16 result is rounded once, where it is stored. The sums of squares have one order
// per (width, groups): a group (or, with fewer than four groups, each of its 4 / groups equal pieces) is summed by
// one wavefront, lanes striding over it, and a group's pieces are added in their order.
#include "common.h"
#include "api.h"

#define GN_THREADS 256
#define GN_WAVES (GN_THREADS / TM_WAVE)

// sums of squares of the units of a row held in `v` (LDS or global), into part[units]
template <typename Load>
__device__ __forceinline__ void unit_sums(Load at, float* part, int glen, int split, int units) {
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int plen = (glen + split - 1) / split;
    for (int u = wave; u < units; u += GN_WAVES) {
        const int g = u / split, i = u - g * split;
        const int lo = g * glen + i * plen;
        const int hi = min(lo + plen, (g + 1) * glen);
        float ss = 0.f;
#pragma unroll 8
        for (int c = lo + lane; c < hi; c += TM_WAVE) {
            const float x = at(c);
            ss += x * x;
        }
        ss = wave_sum(ss);
        if (lane == 0) part[u] = ss;
    }
}

// The groups' 1 / sqrt(mean + eps) from their units' sums, once per group (a root and two divisions per element
// were most of a small step's time), into scale[groups]. Ends with a barrier.
__device__ __forceinline__ void group_scales(const float* part, float* scale, int groups, int split, int glen, float eps) {
    for (int g = threadIdx.x; g < groups; g += GN_THREADS) {
        float ss = part[g * split];
        for (int i = 1; i < split; ++i) ss += part[g * split + i];
        scale[g] = 1.0f / sqrtf(ss / (float)glen + eps);
    }
    __syncthreads();
}

// STAGE: the row of y and both weight vectors are copied into LDS beside the residual row by the first loop, so that
// everything the block needs from memory is asked for at once (one trip instead of four dependent ones: a step of a
// few rows is nothing but those trips); without it (rows too wide for that much LDS) they are read where they are used.
template <typename T, typename WT, bool STAGE>
__global__ __launch_bounds__(GN_THREADS) void group_norm_kernel(float* __restrict__ resid, const T* __restrict__ y,
                                                                const WT* __restrict__ post_w,
                                                                const int* __restrict__ rows,
                                                                const WT* __restrict__ pre_w, T* __restrict__ out,
                                                                int hidden, int groups, int split, float eps) {
    extern __shared__ float lds[];
    float* xs = lds;                                        // the row, [hidden]
    float* ys = lds + hidden;                               // STAGE: y, post_w, pre_w, [hidden] each
    float* pw = lds + 2 * hidden;
    float* qw = lds + 3 * hidden;
    float* part = lds + (STAGE ? 4 : 1) * hidden;           // [groups * split]
    float* scale = part + groups * split;                   // [groups]
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* x = resid + src * hidden;
    const T* yr = y ? y + src * hidden : nullptr;
    const int glen = hidden / groups, units = groups * split;
    // unrolled: the loads of eight rounds are in flight together (left as a loop, every round waits for its own)
#pragma unroll 8
    for (int c = threadIdx.x; c < hidden; c += GN_THREADS) {
        xs[c] = x[c];
        if (STAGE) {
            if (yr) ys[c] = Elem<T>::load(yr + c);
            if (post_w) pw[c] = Elem<WT>::load(post_w + c);
            if (pre_w) qw[c] = Elem<WT>::load(pre_w + c);
        }
    }
    if (STAGE) __syncthreads();
    if (yr) {
        if (post_w) {
            if (STAGE) unit_sums([&](int c) { return ys[c]; }, part, glen, split, units);
            else unit_sums([&](int c) { return Elem<T>::load(yr + c); }, part, glen, split, units);
            __syncthreads();
            group_scales(part, scale, groups, split, glen, eps);
        }
#pragma unroll 8
        for (int c = threadIdx.x; c < hidden; c += GN_THREADS) {
            float d = STAGE ? ys[c] : Elem<T>::load(yr + c);
            if (post_w) d = (STAGE ? pw[c] : Elem<WT>::load(post_w + c)) * (d * scale[c / glen]);
            const float v = xs[c] + d;
            xs[c] = v;
            if (!rows) x[c] = v;
        }
    }
    if (!out) return;
    if (!pre_w) {                               // the sum itself in the result's type (a thread reads what it wrote)
        T* o = out + (size_t)r * hidden;
        for (int c = threadIdx.x; c < hidden; c += GN_THREADS) Elem<T>::store(o + c, xs[c]);
        return;
    }
    __syncthreads();
    unit_sums([&](int c) { return xs[c]; }, part, glen, split, units);
    __syncthreads();
    group_scales(part, scale, groups, split, glen, eps);
    T* o = out + (size_t)r * hidden;
#pragma unroll 8
    for (int c = threadIdx.x; c < hidden; c += GN_THREADS)
        Elem<T>::store(o + c, (STAGE ? qw[c] : Elem<WT>::load(pre_w + c)) * (xs[c] * scale[c / glen]));
}

// The same operation with a row in registers, for rows of at most 4,096 elements in whole groups of four and at most
// eight groups: a thread keeps its (up to four) 4-element pieces of x, y and both weights, which it asked for at once;
// the groups' sums of squares go lane to lane and then through LDS, one barrier per norm. A decode step's norm is a
// chain of dependent steps at a low clock: this one is a third as long as the kernel above.
#define GN_MAX_GROUPS 8
#define GN_PIECES 4

typedef float gn_f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct GnVec;
template <> struct GnVec<float> {
    static __device__ __forceinline__ gn_f32x4 load(const float* p) { return *(const gn_f32x4*)p; }
    static __device__ __forceinline__ void store(float* p, gn_f32x4 v) { *(gn_f32x4*)p = v; }
};
template <> struct GnVec<bf16_t> {
    static __device__ __forceinline__ gn_f32x4 load(const bf16_t* p) {
        const uint2 u = *(const uint2*)p;
        return gn_f32x4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                        __uint_as_float(u.y & 0xffff0000u)};
    }
    static __device__ __forceinline__ void store(bf16_t* p, gn_f32x4 v) {
        uint2 u;
        u.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        u.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *(uint2*)p = u;
    }
};

// 1 / sqrt(mean + eps) of every group from the threads' per-piece sums of squares; sums[i] belongs to group grp[i]
// (-1: no piece). Every thread gets all groups' scales. Lanes are added by the fixed tree of wave_sum, wavefronts in order.
__device__ __forceinline__ void gn_scales(const float (&sums)[GN_PIECES], const int (&grp)[GN_PIECES], int groups, int glen,
                                          float eps, float* red /* [GN_WAVES][GN_MAX_GROUPS] */, float (&scale)[GN_MAX_GROUPS]) {
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    float mine[GN_MAX_GROUPS];
#pragma unroll
    for (int k = 0; k < GN_MAX_GROUPS; ++k) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < GN_PIECES; ++i)
            if (grp[i] == k) v += sums[i];
        mine[k] = k < groups ? wave_sum(v) : 0.f;
    }
    __syncthreads();                            // the last use of red is over
    if (lane == 0) {
#pragma unroll
        for (int k = 0; k < GN_MAX_GROUPS; ++k) red[wave * GN_MAX_GROUPS + k] = mine[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GN_MAX_GROUPS; ++k) {
        float ss = red[k];
#pragma unroll
        for (int w = 1; w < GN_WAVES; ++w) ss += red[w * GN_MAX_GROUPS + k];
        scale[k] = k < groups ? 1.0f / sqrtf(ss / (float)glen + eps) : 0.f;
    }
}

template <typename T, typename WT>
__global__ __launch_bounds__(GN_THREADS) void group_norm_reg_kernel(float* __restrict__ resid, const T* __restrict__ y,
                                                                    const WT* __restrict__ post_w, const int* __restrict__ rows,
                                                                    const WT* __restrict__ pre_w, T* __restrict__ out,
                                                                    int hidden, int groups, float eps) {
    __shared__ float red[GN_WAVES * GN_MAX_GROUPS];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* x = resid + src * hidden;
    const T* yr = y ? y + src * hidden : nullptr;
    const int glen = hidden / groups, pieces = hidden / 4;
    gn_f32x4 xv[GN_PIECES], yv[GN_PIECES], pw[GN_PIECES], qw[GN_PIECES];
    int grp[GN_PIECES];
#pragma unroll
    for (int i = 0; i < GN_PIECES; ++i) {
        const int pc = threadIdx.x + i * GN_THREADS;
        grp[i] = -1;
        xv[i] = yv[i] = pw[i] = qw[i] = gn_f32x4{0.f, 0.f, 0.f, 0.f};
        if (pc < pieces) {
            grp[i] = 4 * pc / glen;             // a piece lies in one group (glen % 4 == 0)
            xv[i] = GnVec<float>::load(x + 4 * pc);
            if (yr) yv[i] = GnVec<T>::load(yr + 4 * pc);
            if (post_w) pw[i] = GnVec<WT>::load(post_w + 4 * pc);
            if (pre_w) qw[i] = GnVec<WT>::load(pre_w + 4 * pc);
        }
    }
    float sums[GN_PIECES], scale[GN_MAX_GROUPS];
    if (yr) {
        if (post_w) {
#pragma unroll
            for (int i = 0; i < GN_PIECES; ++i)
                sums[i] = yv[i][0] * yv[i][0] + yv[i][1] * yv[i][1] + yv[i][2] * yv[i][2] + yv[i][3] * yv[i][3];
            gn_scales(sums, grp, groups, glen, eps, red, scale);
        }
#pragma unroll
        for (int i = 0; i < GN_PIECES; ++i) {
            if (grp[i] < 0) continue;
            float sc = 1.f;
            if (post_w) {
#pragma unroll
                for (int k = 0; k < GN_MAX_GROUPS; ++k)
                    if (grp[i] == k) sc = scale[k];
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) xv[i][k] += post_w ? pw[i][k] * (yv[i][k] * sc) : yv[i][k];
            if (!rows) GnVec<float>::store(x + 4 * (threadIdx.x + i * GN_THREADS), xv[i]);
        }
    }
    if (!out) return;
    if (!pre_w) {
        T* o = out + (size_t)r * hidden;
#pragma unroll
        for (int i = 0; i < GN_PIECES; ++i)
            if (grp[i] >= 0) GnVec<T>::store(o + 4 * (threadIdx.x + i * GN_THREADS), xv[i]);
        return;
    }
#pragma unroll
    for (int i = 0; i < GN_PIECES; ++i)
        sums[i] = xv[i][0] * xv[i][0] + xv[i][1] * xv[i][1] + xv[i][2] * xv[i][2] + xv[i][3] * xv[i][3];
    gn_scales(sums, grp, groups, glen, eps, red, scale);
    T* o = out + (size_t)r * hidden;
#pragma unroll
    for (int i = 0; i < GN_PIECES; ++i) {
        if (grp[i] < 0) continue;
        float sc = 1.f;
#pragma unroll
        for (int k = 0; k < GN_MAX_GROUPS; ++k)
            if (grp[i] == k) sc = scale[k];
        gn_f32x4 v;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = qw[i][k] * (xv[i][k] * sc);
        GnVec<T>::store(o + 4 * (threadIdx.x + i * GN_THREADS), v);
    }
}

static bool gn_in_registers(const float* resid, const void* y, const void* post_w, const void* pre_w, const void* out, int hidden,
                            int groups, int elem, int w_elem) {
    auto ok = [](const void* p, int bytes) { return !p || ((uintptr_t)p % bytes) == 0; };
    return hidden % 4 == 0 && hidden <= 4 * GN_THREADS * GN_PIECES && groups <= GN_MAX_GROUPS && (hidden / groups) % 4 == 0 &&
           ok(resid, 16) && ok(y, 4 * elem) && ok(out, 4 * elem) && ok(post_w, 4 * w_elem) && ok(pre_w, 4 * w_elem);
}

template <typename T, typename WT>
static void launch_group_norm(float* resid, const void* y, const void* post_w, const int* rows, const void* pre_w, void* out, int R,
                              int hidden, int groups, int split, float eps, hipStream_t stream) {
    if (gn_in_registers(resid, y, post_w, pre_w, out, hidden, groups, (int)sizeof(T), (int)sizeof(WT))) {
        group_norm_reg_kernel<T, WT><<<R, GN_THREADS, 0, stream>>>(resid, (const T*)y, (const WT*)post_w, rows, (const WT*)pre_w,
                                                                  (T*)out, hidden, groups, eps);
        return;
    }
    const size_t units = (size_t)groups * split + groups;       // the units' sums and the groups' scales
    const size_t staged = (4 * (size_t)hidden + units) * sizeof(float), plain = ((size_t)hidden + units) * sizeof(float);
    if (staged <= 64 * 1024)
        group_norm_kernel<T, WT, true><<<R, GN_THREADS, staged, stream>>>(resid, (const T*)y, (const WT*)post_w, rows, (const WT*)pre_w,
                                                                         (T*)out, hidden, groups, split, eps);
    else
        group_norm_kernel<T, WT, false><<<R, GN_THREADS, plain, stream>>>(resid, (const T*)y, (const WT*)post_w, rows, (const WT*)pre_w,
                                                                         (T*)out, hidden, groups, split, eps);
}

extern "C" int tm_group_norm(float* resid, const void* y, const void* post_w, const int* rows, const void* pre_w,
                             int w_dtype, void* out, int dtype, int R, int hidden, int groups, float eps,
                             hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (hidden <= 0 || groups <= 0 || hidden % groups || !(eps > 0.f) || !resid) return TM_ERR_ARG;
    if (pre_w && !out) return TM_ERR_ARG;
    if (!y && post_w) return TM_ERR_ARG;
    const int split = groups >= GN_WAVES ? 1 : GN_WAVES / groups;
    const size_t lds = ((size_t)hidden + (size_t)groups * split + groups) * sizeof(float);
    if (lds > 64 * 1024) return TM_ERR_ARG;
    if (dtype == TM_F32 && w_dtype == TM_F32)
        launch_group_norm<float, float>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_BF16)
        launch_group_norm<bf16_t, bf16_t>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_F32)
        launch_group_norm<bf16_t, float>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
