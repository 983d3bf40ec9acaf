// Attention over the paged cache whose heads talk to each other before the softmax:
//   s_h(i, j) = scale * q_h(i) . k(j) + bias[min(i - j, rows - 1)][h]        (a learned bias by distance)
//   s'_h      = sum_g talk[h][g] * s_g                                         (the heads' scores mixed)
//   o_h(i)    = sum_j softmax_j(s'_h(i, .)) v(j)
// Both the bias and the mixing are optional.  Because a head's weights depend on every head's scores against a
// key, one block handles all heads of one token: for 64 keys at a time it forms all scores, mixes them, takes
// the tile into each head's running softmax and adds the tile's values.  Keys are walked from the first key
// the token sees (first_seen_key: all, a window of the last keys, or the token's own chunk), so the order of
// the sums depends on the position alone: not on how the request was cut into steps, nor on the batch.  All
// arithmetic in 32-bit.
//
// cache of one layer: [page][2 (k, v)][Hkv][P][Dc], keys and values both as rows.
#include "common.h"

#define TALK_THREADS 256
#define TALK_MAX_ACC 16          // outputs a thread: Hq * Dv <= 256 * 16

template <typename TA>
__global__ __launch_bounds__(TALK_THREADS) void attention_talk_kernel(
    const TA* __restrict__ q, TA* __restrict__ out, long out_stride, float out_scale, const TA* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tokens, const float* __restrict__ bias, int bias_rows,
    const float* __restrict__ talk, int Hq, int Hkv, int Dk, int Dv, int Dc, int P, float scale, int window) {
    extern __shared__ float sm[];
    float* qs = sm;                               // Hq * Dk
    float* sc = qs + Hq * Dk;                     // Hq * 64 scores
    float* pm = sc + Hq * 64;                     // Hq * 64 weights
    float* ml = pm + Hq * 64;                     // Hq * 2 running maximum and sum
    float* al = ml + Hq * 2;                      // Hq factors of the tile
    float* tk = al + Hq;                          // Hq * Hq (if talk)
    long* voff = (long*)(tk + ((Hq * Hq + 1) & ~1));   // 64 value rows of the tile
    const long t = tokens ? tokens[blockIdx.x] : blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int G = Hq / Hkv;
    const int p = positions[t];
    const int lo = first_seen_key(p, window);
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const long page_stride = 2L * Hkv * P * Dc, plane = (long)Hkv * P * Dc;

    for (int i = tid; i < Hq * Dk; i += TALK_THREADS) {
        const int h = i / Dk, d = i - h * Dk;
        qs[i] = Elem<TA>::load(q + (t * Hq + h) * Dc + d);
    }
    if (talk) for (int i = tid; i < Hq * Hq; i += TALK_THREADS) tk[i] = talk[i];
    for (int h = tid; h < Hq; h += TALK_THREADS) { ml[2 * h] = -INFINITY; ml[2 * h + 1] = 0.f; }
    float acc[TALK_MAX_ACC];
#pragma unroll
    for (int i = 0; i < TALK_MAX_ACC; ++i) acc[i] = 0.f;
    const int n_out = Hq * Dv;
    __syncthreads();

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        const bool seen = j <= p;
        long koff = 0;
        if (seen) {
            const long page = bt[j / P];
            koff = page * page_stride + (long)(j % P) * Dc;
        }
        if (wave == 0) voff[lane] = koff + plane;
        // ---- scores of the tile: thread (wave, lane) takes heads wave, wave + 4, ... against key j
        for (int h = wave; h < Hq; h += TALK_THREADS / 64) {
            float s = 0.f;
            if (seen) {
                const TA* kr = cache + koff + (long)(h / G) * P * Dc;
                const float* qh = qs + h * Dk;
                float dot = 0.f;
                if ((Dk & 3) == 0 && (Dc & 3) == 0) {
                    for (int d = 0; d < Dk; d += 4) {
                        float kv[4];
                        Vec4<TA>::load(kr + d, kv);
                        dot = fmaf(qh[d], kv[0], dot);
                        dot = fmaf(qh[d + 1], kv[1], dot);
                        dot = fmaf(qh[d + 2], kv[2], dot);
                        dot = fmaf(qh[d + 3], kv[3], dot);
                    }
                } else {
                    for (int d = 0; d < Dk; ++d) dot = fmaf(qh[d], Elem<TA>::load(kr + d), dot);
                }
                s = dot * scale;
                if (bias) {
                    const int n = p - j;
                    s += bias[(long)(n < bias_rows ? n : bias_rows - 1) * Hq + h];
                }
            }
            sc[h * 64 + lane] = s;
        }
        __syncthreads();
        // ---- the heads' scores mixed, then the tile joins each head's running softmax
        for (int h = wave; h < Hq; h += TALK_THREADS / 64) {
            float s;
            if (talk) {
                s = 0.f;
                for (int g = 0; g < Hq; ++g) s = fmaf(tk[h * Hq + g], sc[g * 64 + lane], s);
            } else {
                s = sc[h * 64 + lane];
            }
            if (!seen) s = -INFINITY;
            const float m_old = ml[2 * h], l_old = ml[2 * h + 1];
            const float m_new = fmaxf(m_old, wave_max(s));      // finite: key j0 is always seen
            const float a = expf(m_old - m_new);                // exp(-inf) = 0 on the first tile
            const float pj = seen ? expf(s - m_new) : 0.f;
            const float l_new = l_old * a + wave_sum(pj);
            pm[h * 64 + lane] = pj;
            if (lane == 0) { ml[2 * h] = m_new; ml[2 * h + 1] = l_new; al[h] = a; }
        }
        __syncthreads();
        // ---- the tile's values
        const int cnt = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
#pragma unroll
        for (int i = 0; i < TALK_MAX_ACC; ++i) {
            const int o = tid + i * TALK_THREADS;
            if (o < n_out) {
                const int h = o / Dv, d = o - h * Dv;
                const long hv = (long)(h / G) * P * Dc + d;
                const float* ph = pm + h * 64;
                float a = acc[i] * al[h];
                for (int jj = 0; jj < cnt; ++jj) a = fmaf(ph[jj], Elem<TA>::load(cache + voff[jj] + hv), a);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TALK_MAX_ACC; ++i) {
        const int o = tid + i * TALK_THREADS;
        if (o < n_out) {
            const int h = o / Dv;
            Elem<TA>::store(out + t * out_stride + o, acc[i] / ml[2 * h + 1] * out_scale);
        }
    }
}

// q [T, Hq, Dc] (a head's first Dk numbers are read); out: row t at out + t * out_stride, Hq * Dv numbers,
// multiplied by out_scale; bias float32 [bias_rows, Hq] or null; talk float32 [Hq, Hq] or null; tokens: null for
// all T rows, else n_tokens row indices; window as for first_seen_key.
extern "C" int qe_attention_talk(const void* q, void* out, long out_stride, float out_scale, const void* cache,
                                 const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                                 const int* tokens, int n_tokens, const float* bias, int bias_rows, const float* talk,
                                 int Hq, int Hkv, int Dk, int Dv, int Dc, int P, float scale, int window, int dt_a,
                                 hipStream_t stream) {
    QE_REQUIRE(n_tokens >= 0 && Hq > 0 && Hkv > 0 && Dk > 0 && Dv > 0 && P > 0 && max_blocks > 0, "talking attention: bad sizes");
    QE_REQUIRE(Hq % Hkv == 0, "talking attention: %d query heads are no multiple of %d key/value heads", Hq, Hkv);
    QE_REQUIRE(Dc >= Dk && Dc >= Dv, "talking attention: heads of %d and %d numbers in a cache of %d", Dk, Dv, Dc);
    QE_REQUIRE((long)Hq * Dv <= TALK_THREADS * TALK_MAX_ACC, "talking attention: %d heads of %d values are more than %d outputs",
               Hq, Dv, TALK_THREADS * TALK_MAX_ACC);
    QE_REQUIRE(!bias || bias_rows > 0, "talking attention: a bias table without rows");
    QE_REQUIRE(out_stride >= (long)Hq * Dv, "talking attention: output rows overlap");
    if (n_tokens == 0) return 0;
    const size_t floats = (size_t)Hq * Dk + 2 * (size_t)Hq * 64 + 3 * (size_t)Hq + (((size_t)Hq * Hq + 1) & ~(size_t)1);
    const size_t shmem = floats * sizeof(float) + 64 * sizeof(long);
    QE_REQUIRE(shmem <= 150 * 1024, "talking attention: %zu bytes of shared memory", shmem);
#define QE_TALK(TA_)                                                                                                 \
    do {                                                                                                             \
        if (shmem > 48 * 1024)                                                                                       \
            (void)hipFuncSetAttribute((const void*)attention_talk_kernel<TA_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem); \
        attention_talk_kernel<TA_><<<n_tokens, TALK_THREADS, shmem, stream>>>(                                       \
            (const TA_*)q, (TA_*)out, out_stride, out_scale, (const TA_*)cache, positions, tok_seq, block_table,     \
            max_blocks, tokens, bias, bias_rows, talk, Hq, Hkv, Dk, Dv, Dc, P, scale, window);                       \
    } while (0)
    if (dt_a == QE_F32) QE_TALK(float);
    else if (dt_a == QE_BF16) QE_TALK(bf16_t);
    else QE_REQUIRE(false, "talking attention: unknown element type %d", dt_a);
#undef QE_TALK
    QE_LAUNCH_CHECK();
    return 0;
}
