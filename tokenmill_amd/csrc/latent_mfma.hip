// The attention over a shared latent (latent.hip) on MFMA, bfloat16, for the prompt portions and the single tokens of a step.
//
// Every head reads the same cached rows, so a block stages a run of 32 rows in LDS once, as they lie (for the scores) and
// transposed (latent channels x rows, for the results), and works on four tiles of 16 (token, head) pairs with them, one
// wavefront a tile, or two where the latent has more than 128 channels (each with half of them):
//   a prompt tile  : 16 consecutive tokens of one portion; the block's four tiles are four heads;
//   a single token : its heads, 16 a tile (a block takes up to 64 heads); the token's visible rows are dealt in
//                    chunks of one or more runs (aligned to absolute positions; how many runs follows from how far the
//                    model lets a token see, not from the step) to blocks of their own, whose unnormalized results with
//                    their maxima and sums are merged in chunk order: few tokens then fill the chip.
// Per run of rows and tile:
//   S^T = K Q^T      A = rows  [16 rows x 32 d] from LDS, B = Q^T [32 d x 16 pairs] in registers
//   P   = 2^(S * scale * log2 e - m), zero where the row is not visible to the pair, running maximum m and sum l per pair
//   O^T = alpha O^T + C^T P^T   A = latent^T [16 channels x 32 rows] from LDS, B = P^T straight from the S^T accumulators
// Runs are aligned to absolute positions and visited in ascending order, so a pair's result depends on its request's cache
// and its position only.
#include "common.h"
#include "api.h"
#include "attention_prefill_common.h"

#define LM_KEYS 32
#define LM_PAD 16               // staged rows lie 32 bytes more than a multiple of 64 apart: their 16-byte operand loads meet no bank twice
#define LM_VT_STRIDE (LM_KEYS + 8)
#define LM_MAX_CHUNKS 64        // a single token's visible rows are dealt to about this many blocks at most

// WAVES: wavefronts of a block; SPLIT of them share a tile of pairs, each with its own part of the latent's channels (a wide
// latent's results of one tile do not fit a wavefront's registers beside a second wavefront on the SIMD; halved they do, and
// two wavefronts a SIMD hide each other's waits. Both compute the tile's scores). NDT: tiles of 16 latent channels a tile of
// pairs may have (Lk <= 16 NDT). NDC: chunks of 32 channels of a cached row (Dk <= 32 NDC).
template <int WAVES, int NDT, int NDC, int SPLIT>
__global__ __launch_bounds__(64 * WAVES) void attn_latent_mfma_kernel(
    const bf16_t* __restrict__ qa, int q_stride, bf16_t* __restrict__ out, int out_stride, const bf16_t* __restrict__ pool,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ tiles, int head_groups,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, int first_single, float* __restrict__ part_o,
    float* __restrict__ part_ml, int n_chunks, int chunk_runs, int H, int Lk, int Dk, int page, float scale_log2, int window,
    const float* __restrict__ sink) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int DKP = (Dk + 31) / 32 * 32, ndc = DKP / 32;
    const int ks_stride = DKP + LM_PAD;
    bf16_t* Ks = (bf16_t*)lds_raw;                                       // [32][DKP + 8]
    bf16_t* Vt = Ks + LM_KEYS * ks_stride;                               // [Lk rounded up to 16][40]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
    const bool single = tiles == nullptr;
    constexpr int TILES = WAVES / SPLIT, NDTP = NDT / SPLIT;              // tiles of pairs a block; channel tiles a wavefront
    const int d0 = (wave % SPLIT) * NDTP;                                 // this wavefront's first channel tile

    int s, row0, valid, pos0, tile_head;
    if (!single) {
        const int* tl = tiles + (size_t)(blockIdx.x / head_groups) * 4;
        s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
        tile_head = (blockIdx.x % head_groups) * TILES + wave / SPLIT;   // this wavefront's head
    } else {
        row0 = first_single + blockIdx.x / head_groups;
        s = seq_of_token[row0];
        pos0 = positions[row0];
        tile_head = ((blockIdx.x % head_groups) * TILES + wave / SPLIT) * 16;    // its first head
        valid = 1;
    }
    const bool tile_ok = tile_head < H;                                   // wave-uniform
    const int* table = block_tables + (size_t)s * table_width;
    const int last_key = pos0 + valid - 1;
    const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    const int my_pos = single ? pos0 : (pos0 + r < last_key ? pos0 + r : last_key);
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int head = single ? tile_head + r : tile_head;
    const int token = single ? row0 : row0 + r;
    const bool pair_ok = head < H && (single || r < valid);

    // the runs this block visits: all visible ones, or those of its chunk
    int kb_lo = first_key / LM_KEYS, kb_hi = last_key / LM_KEYS;
    if (part_o) {
        const int chunk = kb_lo / chunk_runs + blockIdx.y;
        kb_lo = max(kb_lo, chunk * chunk_runs);
        kb_hi = min(kb_hi, chunk * chunk_runs + chunk_runs - 1);
    }

    PFrag qf[NDC];
#pragma unroll
    for (int c = 0; c < NDC; ++c) {
        const int ch = 32 * c + 8 * g;
        if (tile_ok && pair_ok && ch < Dk)
            qf[c].u = *(const u32x4_t*)(qa + (size_t)token * q_stride + (size_t)head * Dk + ch);
        else
            qf[c].u = u32x4_t{0, 0, 0, 0};
    }
    float m = -INFINITY, l = 0.f;
    f32x4_t o[NDTP];
#pragma unroll
    for (int d = 0; d < NDTP; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const int pieces = DKP / 8;                                           // 16-byte pieces of a staged row
    // Consecutive lanes take consecutive rows (the transposed copy is then written without bank conflicts), so a thread keeps
    // its row through a run: one look into the block table, then all its pieces asked for at once. The pieces of the run
    // after the current one are asked for before the current one is worked on, and stored when that is done.
    constexpr int STEP = 64 * WAVES / LM_KEYS;                            // pieces apart of a thread's consecutive ones
    constexpr int LM_STAGE = (NDC * 4 + STEP - 1) / STEP;                 // 16-byte pieces of a run a thread holds
    // Wide rows leave room for a block or two a CU, and the next run's pieces are asked for before the current run is
    // worked on; narrow rows leave room for four blocks a CU, which hide each other's loads if no registers are held back.
    constexpr bool AHEAD = NDC > 10;
    const int key = threadIdx.x % LM_KEYS, c_first = threadIdx.x / LM_KEYS;
    u32x4_t held[LM_STAGE];
    auto fetch = [&](int kb) {
        const int kj = kb * LM_KEYS + key;
        const bool seen = kj >= first_key && kj <= last_key;
        const bf16_t* src = pool;
        if (seen) src = pool + ((size_t)table[kj / page] * page + kj % page) * Dk;
#pragma unroll
        for (int u = 0; u < LM_STAGE; ++u) {
            const int c8 = c_first + u * STEP;
            held[u] = u32x4_t{0, 0, 0, 0};
            if (seen && 8 * c8 < Dk) held[u] = *(const u32x4_t*)(src + 8 * c8);
        }
    };
    if (AHEAD && kb_lo <= kb_hi) fetch(kb_lo);
    for (int kb = kb_lo; kb <= kb_hi; ++kb) {
        __syncthreads();                                                  // the run before is done with
        if (!AHEAD) fetch(kb);
#pragma unroll
        for (int u = 0; u < LM_STAGE; ++u) {
            const int c8 = c_first + u * STEP;
            if (c8 >= pieces) continue;
            *(u32x4_t*)(Ks + key * ks_stride + 8 * c8) = held[u];
            if (8 * c8 < Lk) {                                            // Lk % 8 == 0: a piece lies wholly inside the latent or not
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Vt[(8 * c8 + 2 * e) * LM_VT_STRIDE + key] = (bf16_t)(held[u][e] & 0xffffu);
                    Vt[(8 * c8 + 2 * e + 1) * LM_VT_STRIDE + key] = (bf16_t)(held[u][e] >> 16);
                }
            }
        }
        __syncthreads();
        if (AHEAD && kb < kb_hi) fetch(kb + 1);                           // in flight while this run is worked on
        if (!tile_ok) continue;
        f32x4_t sc[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int c = 0; c < NDC; ++c) {
            if (c >= ndc) continue;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                PFrag kf;
                kf.u = *(const u32x4_t*)(Ks + (16 * t + r) * ks_stride + 32 * c + 8 * g);
                sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.b, qf[c].b, sc[t], 0, 0, 0);
            }
        }
        const int key0 = kb * LM_KEYS;
        float sv[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kj = key0 + 16 * t + 4 * g + i;
                float v = sc[t][i] * scale_log2;
                if (kj > my_pos || kj < my_lo) v = -INFINITY;
                sv[t][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, TM_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, TM_WAVE));
        const float m_new = fmaxf(m, mx);
        const float ref = m_new == -INFINITY ? 0.f : m_new;               // no row seen yet: every weight is zero
        const float alpha = __builtin_amdgcn_exp2f(m - ref);
        m = m_new;
        float pr[2][4], sum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pr[t][i] = __builtin_amdgcn_exp2f(sv[t][i] - ref);
                sum += pr[t][i];
            }
        l = l * alpha + sum;
        PFrag pt;
        pt.u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                       pk_bf16(pr[1][2], pr[1][3])};
#pragma unroll
        for (int d = 0; d < NDTP; ++d) {
            if (16 * (d0 + d) >= Lk) continue;                            // wave-uniform
            o[d] *= alpha;
            const bf16_t* vrow = Vt + (16 * (d0 + d) + r) * LM_VT_STRIDE + 4 * g;
            const u32x2_t v0 = *(const u32x2_t*)vrow, v1 = *(const u32x2_t*)(vrow + 16);
            PFrag vf;
            vf.u = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
            o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[d], 0, 0, 0);
        }
    }
    if (!tile_ok) return;
    float total = l;
    total += __shfl_xor(total, 16, TM_WAVE);
    total += __shfl_xor(total, 32, TM_WAVE);
    if (!pair_ok) return;
    if (part_o) {                                                         // a chunk's share: as it is, with its maximum and sum
        const size_t at = ((size_t)(row0 - first_single) * H + head) * n_chunks + blockIdx.y;
        if (g == 0 && wave % SPLIT == 0) {
            part_ml[2 * at] = m;
            part_ml[2 * at + 1] = total;
        }
        float* dst = part_o + at * Lk;
#pragma unroll
        for (int d = 0; d < NDTP; ++d) {
            const int ch = 16 * (d0 + d) + 4 * g;
            if (ch < Lk) *(f32x4_t*)(dst + ch) = o[d];
        }
        return;
    }
    // the sink of the pair's head: one more term of the denominator, with no row behind it (m is a power of two's exponent)
    if (sink) total += __builtin_amdgcn_exp2f(sink[head] * 1.4426950408889634f - m);
    const float inv = 1.0f / total;
    bf16_t* dst = out + (size_t)token * out_stride + (size_t)head * Lk;
#pragma unroll
    for (int d = 0; d < NDTP; ++d) {
        const int ch = 16 * (d0 + d) + 4 * g;
        if (ch < Lk) *(u32x2_t*)(dst + ch) = u32x2_t{pk_bf16(o[d][0] * inv, o[d][1] * inv), pk_bf16(o[d][2] * inv, o[d][3] * inv)};
    }
}

// out[token, head] = sum_y part_o[y] 2^(m_y - M) / sum_y l_y 2^(m_y - M), M = max_y m_y, chunks y in their order; a chunk
// without a visible row (m = -inf, zeros in part_o) weighs nothing. With a sink, L also holds 2^(sink[h] log2 e - M) and M is
// at least the sink's exponent.
__global__ __launch_bounds__(128) void attn_latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                bf16_t* __restrict__ out, int out_stride, int first_single, int H,
                                                                int Lk, int n_chunks, const float* __restrict__ sink) {
    extern __shared__ float w_s[];                                        // a chunk's weight 2^(m_y - M) / L
    const int pair = blockIdx.x, t = pair / H, h = pair % H;
    const float* ml = part_ml + (size_t)pair * n_chunks * 2;
    if (threadIdx.x < TM_WAVE) {                                          // one wavefront: maximum, sum, weights
        float M = -INFINITY;
        for (int y = threadIdx.x; y < n_chunks; y += TM_WAVE) M = fmaxf(M, ml[2 * y]);
        M = wave_max(M);
        const float sk = sink ? sink[h] * 1.4426950408889634f : -INFINITY;
        M = fmaxf(M, sk);
        float L = sink ? __builtin_amdgcn_exp2f(sk - M) : 0.f;
        for (int y0 = 0; y0 < n_chunks; y0 += TM_WAVE) {                  // the chunks' sums in their order, 64 at a time
            const int y = y0 + threadIdx.x;
            const float e = (y < n_chunks && ml[2 * y] != -INFINITY) ? ml[2 * y + 1] * __builtin_amdgcn_exp2f(ml[2 * y] - M) : 0.f;
            L += wave_sum(e);
        }
        const float inv = 1.0f / L;
        for (int y = threadIdx.x; y < n_chunks; y += TM_WAVE)
            w_s[y] = ml[2 * y] != -INFINITY ? __builtin_amdgcn_exp2f(ml[2 * y] - M) * inv : 0.f;
    }
    __syncthreads();
    bf16_t* dst = out + (size_t)(first_single + t) * out_stride + (size_t)h * Lk;
    const float* po = part_o + (size_t)pair * n_chunks * Lk;
    for (int c = 4 * threadIdx.x; c < Lk; c += 4 * 128) {                 // Lk % 8 == 0; a chunk without rows holds zeros
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int y = 0; y < n_chunks; ++y) acc += *(const f32x4_t*)(po + (size_t)y * Lk + c) * w_s[y];
        *(u32x2_t*)(dst + c) = u32x2_t{pk_bf16(acc[0], acc[1]), pk_bf16(acc[2], acc[3])};
    }
}

static size_t lm_lds_bytes(int Lk, int Dk) {
    const int DKP = (Dk + 31) / 32 * 32;
    return (size_t)LM_KEYS * (DKP + LM_PAD) * 2 + (size_t)((Lk + 15) / 16 * 16) * LM_VT_STRIDE * 2;
}

// bfloat16; Dk and Lk multiples of 8 (16-byte pieces of a row lie inside the latent or outside it), rows of up to 704
// channels with up to 512 of latent.
extern "C" int tm_attn_latent_mfma_takes(int Lk, int Dk, int q_stride, int out_stride) {
    return Lk > 0 && Lk <= 512 && Dk >= Lk && Dk <= 704 && Lk % 8 == 0 && Dk % 8 == 0 && q_stride % 8 == 0 && out_stride % 4 == 0;
}

// Runs of 32 rows in a chunk of a single token's rows, for a model whose tokens see at most `bound` rows (its window or its
// longest context): one, or as many as keep the chunks at about LM_MAX_CHUNKS.
extern "C" int tm_attn_latent_chunk_runs(int bound) {
    const int runs = (bound + LM_KEYS - 1) / LM_KEYS;
    return runs <= LM_MAX_CHUNKS ? 1 : (runs + LM_MAX_CHUNKS - 1) / LM_MAX_CHUNKS;
}

// Chunks of `chunk_runs` runs that a single token's visible rows can fall into when it sees at most `most_rows` of them.
extern "C" int tm_attn_latent_chunks(int most_rows, int chunk_runs) {
    if (chunk_runs <= 0) return 0;
    return (most_rows + LM_KEYS * chunk_runs - 1) / (LM_KEYS * chunk_runs) + 1;
}

struct LmArgs {
    const bf16_t* qa; int q_stride; bf16_t* out; int out_stride; const bf16_t* pool; const int* block_tables; int table_width;
    const int* tiles; int head_groups; const int* seq_of_token; const int* positions; int first_single; float* part_o;
    float* part_ml; int n_chunks; int chunk_runs; int H, Lk, Dk, page; float scale_log2; int window; const float* sink;
};

template <int WAVES, int NDT, int NDC, int SPLIT>
static int lm_launch(dim3 grid, size_t lds, hipStream_t stream, const LmArgs& a) {
    auto kernel = attn_latent_mfma_kernel<WAVES, NDT, NDC, SPLIT>;
    static size_t allowed = 64 * 1024;                                   // per instantiation: the most LDS asked for so far
    if (lds > allowed) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        allowed = lds;
    }
    kernel<<<grid, 64 * WAVES, lds, stream>>>(a.qa, a.q_stride, a.out, a.out_stride, a.pool, a.block_tables, a.table_width, a.tiles,
                                              a.head_groups, a.seq_of_token, a.positions, a.first_single, a.part_o, a.part_ml,
                                              a.n_chunks, a.chunk_runs, a.H, a.Lk, a.Dk, a.page, a.scale_log2, a.window,
                                              a.part_o ? nullptr : a.sink);      // a chunk's share meets the sink in the merge, once
    return TM_OK;
}

// a latent of more than 128 channels: eight wavefronts a block, two a tile of pairs; four tiles a block either way
static int lm_pick(dim3 grid, size_t lds, hipStream_t stream, const LmArgs& a) {
    const int ndt = (a.Lk + 15) / 16, ndc = (a.Dk + 31) / 32;
#define LM_ROW(WAVES_, NDT_, SPLIT_)                                                         \
    if (ndc <= 4) return lm_launch<WAVES_, NDT_, 4, SPLIT_>(grid, lds, stream, a);           \
    if (ndc <= 10) return lm_launch<WAVES_, NDT_, 10, SPLIT_>(grid, lds, stream, a);         \
    return lm_launch<WAVES_, NDT_, 22, SPLIT_>(grid, lds, stream, a);
    if (ndt <= 8) { LM_ROW(4, 8, 1) }
    if (ndt <= 16) { LM_ROW(8, 16, 2) }
    LM_ROW(8, 32, 2)
#undef LM_ROW
}

// The prompt tiles of a step (tiles [n_tiles][4] as for tm_attn_prefill_mfma) or its single tokens (rows first_single ..
// first_single + n_single - 1; part_o [n_single * H, n_chunks, Lk] and part_ml [n_single * H, n_chunks, 2] are 32-bit
// scratch, chunk_runs = tm_attn_latent_chunk_runs(the model's bound), n_chunks = tm_attn_latent_chunks(the most rows a token
// of the call can see, chunk_runs)); one of the two per call.
extern "C" int tm_attn_latent_mfma(const void* qa, int q_stride, void* out, int out_stride, const void* pool,
                                   const int* block_tables, int table_width, const int* tiles, int n_tiles,
                                   const int* seq_of_token, const int* positions, int first_single, int n_single, float* part_o,
                                   float* part_ml, int n_chunks, int chunk_runs, int H, int Lk, int Dk, int page, float scale,
                                   int window, const float* sink, hipStream_t stream) {
    if ((n_tiles > 0) == (n_single > 0)) return (n_tiles == 0 && n_single == 0) ? TM_OK : TM_ERR_ARG;
    if (!qa || !out || !pool || !block_tables || H <= 0 || page <= 0 || window < 0 || table_width <= 0 ||
        !tm_attn_latent_mfma_takes(Lk, Dk, q_stride, out_stride) || ((uintptr_t)qa % 16) || ((uintptr_t)out % 8) ||
        ((uintptr_t)pool % 16) || (long long)q_stride < (long long)H * Dk || (long long)out_stride < (long long)H * Lk ||
        (n_tiles > 0 && !tiles) ||
        (n_single > 0 && (!seq_of_token || !positions || !part_o || !part_ml || n_chunks <= 0 || n_chunks > 65535 || chunk_runs <= 0 ||
                          ((uintptr_t)part_o % 16))))
        return TM_ERR_ARG;
    LmArgs a{(const bf16_t*)qa, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)pool, block_tables, table_width,
             n_tiles > 0 ? tiles : nullptr, 1, seq_of_token, positions, first_single, nullptr, nullptr, n_chunks, chunk_runs,
             H, Lk, Dk, page, scale * 1.4426950408889634f, window, sink};
    const size_t lds = lm_lds_bytes(Lk, Dk);
    int rc;
    if (n_tiles > 0) {
        a.head_groups = (H + 3) / 4;
        const long long blocks = (long long)n_tiles * a.head_groups;
        if (blocks > 0x7fffffffLL) return TM_ERR_ARG;
        rc = lm_pick(dim3((unsigned)blocks), lds, stream, a);
    } else {
        a.head_groups = (H + 63) / 64;                                    // four wavefronts stage a run together; each takes 16 heads
        a.part_o = part_o;
        a.part_ml = part_ml;
        const long long blocks = (long long)n_single * a.head_groups;
        if (blocks > 0x7fffffffLL) return TM_ERR_ARG;
        rc = lm_pick(dim3((unsigned)blocks, n_chunks), lds, stream, a);
        if (rc == TM_OK) {
            TM_CHECK_LAUNCH();
            attn_latent_merge_kernel<<<n_single * H, 128, (size_t)n_chunks * sizeof(float), stream>>>(part_o, part_ml, (bf16_t*)out, out_stride, first_single, H, Lk,
                                                                       n_chunks, sink);
        }
    }
    if (rc != TM_OK) return rc;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
