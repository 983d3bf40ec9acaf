// Attention over the paged cache whose heads talk to each other before the softmax:
//   s_h(i, j) = scale * q_h(i) . k(j) + bias[min(i - j, rows - 1)][h]        (a learned bias by distance)
//   s'_h      = sum_g talk[h][g] * s_g                                         (the heads' scores mixed)
//   o_h(i)    = sum_j softmax_j(s'_h(i, .)) v(j)
// Both the bias and the mixing are optional.  Because a head's weights depend on every head's scores against a
// key, one block handles all heads of one token.  Keys are walked 64 at a time from the first key the token sees
// (first_seen_key: all, a window of the last keys, or the token's own chunk).  A tile of 64 keys goes through a
// staging buffer in shared memory in stages, each brought in by contiguous loads and converted to 32-bit, the loads
// of the next stage (or of the next tile's first) in flight while the block computes on the present one:
//   - the key rows of as many key/value heads as fit (rows padded so that a lane per key reads its row without bank
//     conflicts): every wave takes query heads in turn, a lane per key, for the dot products; the biases of a
//     tile are loaded a tile ahead;
//   - after the last stage of keys the heads' scores are mixed and the tile joins each head's running softmax (a
//     wave per head);
//   - the value rows of all key/value heads for as many of the tile's keys as fit: a thread per four neighbouring
//     output numbers adds the stage's values.
// With KS > 1 the tiles of a token are dealt to KS blocks in turn; each leaves its maxima, sums and accumulators in a
// workspace and attention_talk_merge_kernel weighs and adds them in the order of the splits.  The order of the sums
// depends on the position and KS alone: not on how the request was cut into steps.  All arithmetic in 32-bit.
//
// cache of one layer: [page][2 (k, v)][Hkv][P][Dc], keys and values both as rows, zeros beyond a head's own numbers,
// Dc a multiple of 4.
#include "common.h"

#define TALK_THREADS 256
#define TALK_MAX_ACC 8           // groups of four outputs a thread: Hq * ceil(Dv / 4) <= 256 * 8
#define TALK_ROWS_ACC 2          // the same in the kernel for many rows, which holds them for every row of the block
#define TALK_MAX_SPLITS 16
#define TALK_ROWS 4              // rows a block of the kernel for many rows

// Four consecutive elements as they lie in memory, and as four floats.
template <typename T> struct Raw4;
template <> struct Raw4<float> {
    typedef float4 R;
    static __device__ __forceinline__ R load(const float* p) { return *(const float4*)p; }
    static __device__ __forceinline__ R zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ float4 widen(R r) { return r; }
};
template <> struct Raw4<bf16_t> {
    typedef uint2 R;
    static __device__ __forceinline__ R load(const bf16_t* p) { return *(const uint2*)p; }
    static __device__ __forceinline__ R zero() { return make_uint2(0u, 0u); }
    static __device__ __forceinline__ float4 widen(R r) {
        return make_float4(bf16_bits_to_float(r.x & 0xffffu), bf16_bits_to_float(r.x >> 16),
                           bf16_bits_to_float(r.y & 0xffffu), bf16_bits_to_float(r.y >> 16));
    }
};

struct TalkLayout {              // offsets into shared memory, in floats (all multiples of 4)
    int rs_q, ls_k, ls_v, stage, sc, pm, small, total;
};

__host__ __device__ __forceinline__ TalkLayout talk_layout(int Hq, int Hkv, int Dk, int Dv, int HGk, int KPS) {
    TalkLayout L;
    L.rs_q = (Dk + 3) & ~3;
    L.ls_k = L.rs_q + (((L.rs_q >> 2) & 1) ? 0 : 4);      // an odd number of 16-byte pieces a row
    L.ls_v = (Dv + 3) & ~3;
    const int a = HGk * 64 * L.ls_k, b = Hkv * KPS * L.ls_v;
    L.stage = 256 + Hq * L.rs_q;                           // (256 floats = twice 64 offsets of 8 bytes come first)
    L.sc = L.stage + (a > b ? a : b);
    L.pm = L.sc + Hq * 64;
    L.small = L.pm + Hq * 64;
    L.total = L.small + ((3 * Hq + Hq * Hq + 3) & ~3);
    return L;
}

// A stage of keys: the key rows of `hg` key/value heads from g0 for the tile's 64 keys (row gl * 64 + jj).  A stage of
// values: the value rows of all key/value heads for KPS of the tile's keys from k0 (row gl * KPS + jl), so that every
// thread has work in every stage.  talk_fetch starts the loads of a stage into registers (NV pieces of four numbers a
// thread; keys that are not seen, offset < 0, become zeros); talk_commit writes them to the staging buffer in 32-bit.
// Between the two the block computes on the stage before.
// item[u]: (row of the stage << 8) | piece of the row, for the thread's u-th piece of a full stage; -1: beyond it
template <int NV>
__device__ __forceinline__ void talk_items(int (&item)[NV], int rows, int vec_per_row) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = threadIdx.x + u * TALK_THREADS;
        item[u] = i < rows * vec_per_row ? ((i / vec_per_row) << 8) | (i % vec_per_row) : -1;
    }
}

// rows: of this stage (<= those of a full one); a row's key is k0 + (row & (2^kshift - 1)), its head g0 + (row >> kshift)
template <typename TA, int NV>
__device__ __forceinline__ void talk_fetch(typename Raw4<TA>::R (&regs)[NV], const int (&item)[NV],
                                           const TA* __restrict__ plane, const long* koff, int g0, int rows, int kshift,
                                           int k0, long head_stride) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        typename Raw4<TA>::R r = Raw4<TA>::zero();
        const int rr = item[u] >> 8;
        if (item[u] >= 0 && rr < rows) {
            const long off = koff[k0 + (rr & ((1 << kshift) - 1))];
            if (off >= 0) r = Raw4<TA>::load(plane + off + (long)(g0 + (rr >> kshift)) * head_stride + (item[u] & 255) * 4);
        }
        regs[u] = r;
    }
}

template <typename TA, int NV>
__device__ __forceinline__ void talk_commit(const typename Raw4<TA>::R (&regs)[NV], const int (&item)[NV],
                                            float* stage, int rows, int ls) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int rr = item[u] >> 8;
        if (item[u] >= 0 && rr < rows)
            *(float4*)(stage + (long)rr * ls + (item[u] & 255) * 4) = Raw4<TA>::widen(regs[u]);
    }
}

#define TALK_BIAS_PRE 8          // a thread's first heads' biases for the next tile are loaded a tile ahead

template <typename TA, int NV>
__global__ __launch_bounds__(TALK_THREADS) void attention_talk_kernel(
    const TA* __restrict__ q, TA* __restrict__ out, long out_stride, float out_scale, const TA* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tokens, const float* __restrict__ bias, int bias_rows,
    const float* __restrict__ talk, int Hq, int Hkv, int Dk, int Dv, int Dc, int P, float scale, int window,
    int KS, int HGk, int kps_shift, float* __restrict__ ws) {
    extern __shared__ __align__(16) float sm[];
    const int KPS = 1 << kps_shift;
    const TalkLayout L = talk_layout(Hq, Hkv, Dk, Dv, HGk, KPS);
    long* koff = (long*)sm;                       // twice 64 key rows: this tile's and the next one's (-1: not seen)
    float* qs = sm + 256;                         // Hq rows of rs_q
    float* stage = sm + L.stage;
    float* sc = sm + L.sc;                        // Hq * 64 scores
    float* pm = sm + L.pm;                        // Hq * 64 weights
    float* ml = sm + L.small;                     // Hq * 2 running maximum and sum
    float* al = ml + 2 * Hq;                      // Hq factors of the tile
    float* tk = al + Hq;                          // Hq * Hq (if talk)
    const long t = tokens ? tokens[blockIdx.x] : blockIdx.x;
    const int split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int G = Hq / Hkv;
    const int p = positions[t];
    const int lo = first_seen_key(p, window);
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const long page_stride = 2L * Hkv * P * Dc, plane = (long)Hkv * P * Dc, head_stride = (long)P * Dc;
    const int n_out = Hq * Dv;
    const int nK = (Hkv + HGk - 1) / HGk, nS = nK + (64 >> kps_shift);           // stages of a tile: keys, then values
    const int vpr_k = L.rs_q >> 2, vpr_v = L.ls_v >> 2;

    for (int i = tid; i < Hq * L.rs_q; i += TALK_THREADS) {
        const int h = i / L.rs_q, d = i - h * L.rs_q;
        qs[i] = d < Dk ? Elem<TA>::load(q + (t * Hq + h) * Dc + d) : 0.f;
    }
    if (talk) for (int i = tid; i < Hq * Hq; i += TALK_THREADS) tk[i] = talk[i];
    for (int h = tid; h < Hq; h += TALK_THREADS) { ml[2 * h] = -INFINITY; ml[2 * h + 1] = 0.f; }
    float4 acc[TALK_MAX_ACC];
    int hd[TALK_MAX_ACC];                          // a group's head and first column
#pragma unroll
    for (int i = 0; i < TALK_MAX_ACC; ++i) {
        acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        const int o = tid + i * TALK_THREADS;
        const int h = o < Hq * vpr_v ? o / vpr_v : Hq;
        hd[i] = (h << 16) | (h < Hq ? (o - h * vpr_v) * 4 : 0);
    }
    typename Raw4<TA>::R regs[NV];
    int item_k[NV], item_v[NV];
    talk_items<NV>(item_k, HGk * 64, vpr_k);
    talk_items<NV>(item_v, Hkv * KPS, vpr_v);
    float bpre[TALK_BIAS_PRE];                     // biases of heads wave, wave + 4, ... against this lane's key

    int j0 = lo + 64 * split, par = 0;
    if (j0 <= p) {
        const int j = j0 + lane;
        if (wave == 0) koff[lane] = j <= p ? (long)bt[j / P] * page_stride + (long)(j % P) * Dc : -1L;
#pragma unroll
        for (int i = 0; i < TALK_BIAS_PRE; ++i) {
            const int h = wave + 4 * i, n = p - j;
            bpre[i] = (bias && j <= p && h < Hq) ? bias[(long)(n < bias_rows ? n : bias_rows - 1) * Hq + h] : 0.f;
        }
        __syncthreads();
        talk_fetch<TA, NV>(regs, item_k, cache, koff, 0, (Hkv < HGk ? Hkv : HGk) * 64, 6, 0, head_stride);
    }
    for (; j0 <= p; j0 += 64 * KS, par ^= 1) {
        const long* ko = koff + par * 64;
        long* kn = koff + (par ^ 1) * 64;
        const int jn = j0 + 64 * KS;
        const bool more = jn <= p;
        const int j = j0 + lane;
        const bool seen = j <= p;
        if (wave == 0) kn[lane] = jn + lane <= p ? (long)bt[(jn + lane) / P] * page_stride + (long)((jn + lane) % P) * Dc : -1L;
        float bnow[TALK_BIAS_PRE];
#pragma unroll
        for (int i = 0; i < TALK_BIAS_PRE; ++i) bnow[i] = bpre[i];
        for (int s = 0; s < nS; ++s) {
            const bool is_v = s >= nK;
            const int g0 = is_v ? 0 : s * HGk;
            const int hg = is_v ? Hkv : (Hkv - g0 < HGk ? Hkv - g0 : HGk);
            const int k0 = is_v ? (s - nK) << kps_shift : 0;
            __syncthreads();                                 // (the stage before has been read)
            if (is_v) talk_commit<TA, NV>(regs, item_v, stage, Hkv * KPS, L.ls_v);
            else talk_commit<TA, NV>(regs, item_k, stage, hg * 64, L.ls_k);
            if (s + 1 < nS) {                                // the next stage's loads fly while this one is computed on
                if (s + 1 >= nK) {
                    talk_fetch<TA, NV>(regs, item_v, cache + plane, ko, 0, Hkv * KPS, kps_shift, (s + 1 - nK) << kps_shift,
                                       head_stride);
                } else {
                    const int n0 = (s + 1) * HGk;
                    talk_fetch<TA, NV>(regs, item_k, cache, ko, n0, (Hkv - n0 < HGk ? Hkv - n0 : HGk) * 64, 6, 0, head_stride);
                }
            } else if (more) {
                talk_fetch<TA, NV>(regs, item_k, cache, kn, 0, (Hkv < HGk ? Hkv : HGk) * 64, 6, 0, head_stride);
#pragma unroll
                for (int i = 0; i < TALK_BIAS_PRE; ++i) {
                    const int h = wave + 4 * i, n = p - (jn + lane);
                    bpre[i] = (bias && n >= 0 && h < Hq) ? bias[(long)(n < bias_rows ? n : bias_rows - 1) * Hq + h] : 0.f;
                }
            }
            __syncthreads();
            if (!is_v) {
                // ---- scores: thread (wave, lane) takes heads wave, wave + 4, ... of the staged key heads against key j
#pragma unroll
                for (int i = 0; i < TALK_BIAS_PRE; ++i) {
                    const int h = wave + 4 * i, gk = h / G;
                    if (h < Hq && gk >= g0 && gk < g0 + hg) {
                        const float4* kr = (const float4*)(stage + (long)((gk - g0) * 64 + lane) * L.ls_k);
                        const float4* qh = (const float4*)(qs + h * L.rs_q);
                        float d0 = 0.f, d1 = 0.f;
#pragma unroll 4
                        for (int d = 0; d < vpr_k; ++d) {
                            const float4 a = qh[d], b = kr[d];
                            d0 = fmaf(a.x, b.x, d0); d1 = fmaf(a.y, b.y, d1);
                            d0 = fmaf(a.z, b.z, d0); d1 = fmaf(a.w, b.w, d1);
                        }
                        sc[h * 64 + lane] = (d0 + d1) * scale + bnow[i];
                    }
                }
                for (int h = wave + 4 * TALK_BIAS_PRE; h < Hq; h += TALK_THREADS / 64) {      // (more than 32 heads)
                    const int gk = h / G;
                    if (gk < g0 || gk >= g0 + hg) continue;
                    const float4* kr = (const float4*)(stage + (long)((gk - g0) * 64 + lane) * L.ls_k);
                    const float4* qh = (const float4*)(qs + h * L.rs_q);
                    float d0 = 0.f, d1 = 0.f;
                    for (int d = 0; d < vpr_k; ++d) {
                        const float4 a = qh[d], b = kr[d];
                        d0 = fmaf(a.x, b.x, d0); d1 = fmaf(a.y, b.y, d1);
                        d0 = fmaf(a.z, b.z, d0); d1 = fmaf(a.w, b.w, d1);
                    }
                    float sv = (d0 + d1) * scale;
                    if (bias && seen) {
                        const int n = p - j;
                        sv += bias[(long)(n < bias_rows ? n : bias_rows - 1) * Hq + h];
                    }
                    sc[h * 64 + lane] = sv;
                }
                if (s == nK - 1) {
                    __syncthreads();
                    // ---- the heads' scores mixed, then the tile joins each head's running softmax
                    for (int h = wave; h < Hq; h += TALK_THREADS / 64) {
                        float sv;
                        if (talk) {
                            sv = 0.f;
                            for (int g = 0; g < Hq; ++g) sv = fmaf(tk[h * Hq + g], sc[g * 64 + lane], sv);
                        } else {
                            sv = sc[h * 64 + lane];
                        }
                        if (!seen) sv = -INFINITY;
                        const float m_old = ml[2 * h], l_old = ml[2 * h + 1];
                        const float m_new = fmaxf(m_old, wave_max(sv));     // finite: key j0 is always seen
                        const float a = expf(m_old - m_new);                // exp(-inf) = 0 on the first tile
                        const float pj = seen ? expf(sv - m_new) : 0.f;
                        const float l_new = l_old * a + wave_sum(pj);
                        pm[h * 64 + lane] = pj;
                        if (lane == 0) { ml[2 * h] = m_new; ml[2 * h + 1] = l_new; al[h] = a; }
                    }
                }
            } else {
                // ---- the stage's values (unseen keys: zeros with weight zero)
#pragma unroll
                for (int i = 0; i < TALK_MAX_ACC; ++i) {
                    const int h = hd[i] >> 16;
                    if (h < Hq) {
                        const float* vs = stage + (long)(h / G) * KPS * L.ls_v + (hd[i] & 0xffff);
                        const float4* ph = (const float4*)(pm + h * 64 + k0);
                        const float f = k0 == 0 ? al[h] : 1.f;
                        float4 a = make_float4(acc[i].x * f, acc[i].y * f, acc[i].z * f, acc[i].w * f);
#pragma unroll 2
                        for (int jj = 0; jj < (KPS >> 2); ++jj) {
                            const float4 w = ph[jj];
                            const float wa[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float4 vv = *(const float4*)(vs + (long)(jj * 4 + e) * L.ls_v);
                                a.x = fmaf(wa[e], vv.x, a.x); a.y = fmaf(wa[e], vv.y, a.y);
                                a.z = fmaf(wa[e], vv.z, a.z); a.w = fmaf(wa[e], vv.w, a.w);
                            }
                        }
                        acc[i] = a;
                    }
                }
            }
        }
    }
    __syncthreads();
    if (KS == 1) {
#pragma unroll
        for (int i = 0; i < TALK_MAX_ACC; ++i) {
            const int h = hd[i] >> 16, d = hd[i] & 0xffff;
            if (h < Hq) {
                const float f = out_scale / ml[2 * h + 1];
                const float a[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
                for (int e = 0; e < 4; ++e)
                    if (d + e < Dv) Elem<TA>::store(out + t * out_stride + h * Dv + d + e, a[e] * f);
            }
        }
        return;
    }
    float* w = ws + ((long)blockIdx.x * KS + split) * (2 * Hq + n_out);
    for (int i = tid; i < 2 * Hq; i += TALK_THREADS) w[i] = ml[i];
#pragma unroll
    for (int i = 0; i < TALK_MAX_ACC; ++i) {
        const int h = hd[i] >> 16, d = hd[i] & 0xffff;
        if (h < Hq) {
            const float a[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
            for (int e = 0; e < 4; ++e)
                if (d + e < Dv) w[2 * Hq + h * Dv + d + e] = a[e];
        }
    }
}

// ---- several rows a block ------------------------------------------------------------------------------------
// For portions of prompts: a block takes R neighbouring rows of the flat batch.  Rows of one request whose first seen
// key is the same (one chunk, or no window) are walked together over the keys up to the last row's position, so that
// a stage of keys or values is brought in once for all of them, a key's numbers are read once for R dot products, and a
// value's once for R sums; every row masks the keys behind its own position.  Rows of the block that belong
// elsewhere (another request, the next chunk) get a pass of their own.  Everything else as in the kernel above.
struct TalkRowsLayout { int stage, sc, pm, small, total; };

__host__ __device__ __forceinline__ TalkRowsLayout talk_rows_layout(const TalkLayout& L1, int R, int Hq) {
    TalkRowsLayout L;
    const int stage_floats = L1.sc - L1.stage;
    L.stage = 256 + R * Hq * L1.rs_q;
    L.sc = L.stage + stage_floats;
    L.pm = L.sc + R * Hq * 64;
    L.small = L.pm + R * Hq * 64;
    L.total = L.small + ((3 * R * Hq + Hq * Hq + 3) & ~3);
    return L;
}

template <typename TA, int NV, int R>
__global__ __launch_bounds__(TALK_THREADS) void attention_talk_rows_kernel(
    const TA* __restrict__ q, TA* __restrict__ out, long out_stride, float out_scale, const TA* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int T, const float* __restrict__ bias, int bias_rows, const float* __restrict__ talk, int Hq,
    int Hkv, int Dk, int Dv, int Dc, int P, float scale, int window, int KS, int HGk, int kps_shift,
    float* __restrict__ ws) {
    extern __shared__ __align__(16) float sm[];
    const int KPS = 1 << kps_shift;
    const TalkLayout L = talk_layout(Hq, Hkv, Dk, Dv, HGk, KPS);
    const TalkRowsLayout LR = talk_rows_layout(L, R, Hq);
    long* koff = (long*)sm;
    float* qs = sm + 256;                         // R * Hq rows of rs_q
    float* stage = sm + LR.stage;
    float* sc = sm + LR.sc;                       // R * Hq * 64 scores
    float* pm = sm + LR.pm;                       // R * Hq * 64 weights
    float* ml = sm + LR.small;                    // R * Hq * 2 running maximum and sum
    float* al = ml + 2 * R * Hq;                  // R * Hq factors of the tile
    float* tk = al + R * Hq;                      // Hq * Hq (if talk)
    const int split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int G = Hq / Hkv;
    const long page_stride = 2L * Hkv * P * Dc, plane = (long)Hkv * P * Dc, head_stride = (long)P * Dc;
    const int n_out = Hq * Dv;
    const int nK = (Hkv + HGk - 1) / HGk, nS = nK + (64 >> kps_shift);
    const int vpr_k = L.rs_q >> 2, vpr_v = L.ls_v >> 2;
    const long row0 = (long)blockIdx.x * R;

    int pr[R], sq[R], lo_r[R];                     // (the same in every thread)
    unsigned todo = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        pr[r] = 0; sq[r] = -1; lo_r[r] = 0;
        if (row0 + r < T) {
            pr[r] = positions[row0 + r];
            sq[r] = tok_seq[row0 + r];
            lo_r[r] = first_seen_key(pr[r], window);
            todo |= 1u << r;
        }
    }
    if (talk) for (int i = tid; i < Hq * Hq; i += TALK_THREADS) tk[i] = talk[i];
    int hd[TALK_ROWS_ACC];
#pragma unroll
    for (int i = 0; i < TALK_ROWS_ACC; ++i) {
        const int o = tid + i * TALK_THREADS;
        const int h = o < Hq * vpr_v ? o / vpr_v : Hq;
        hd[i] = (h << 16) | (h < Hq ? (o - h * vpr_v) * 4 : 0);
    }
    int item_k[NV], item_v[NV];
    talk_items<NV>(item_k, HGk * 64, vpr_k);
    talk_items<NV>(item_v, Hkv * KPS, vpr_v);
    typename Raw4<TA>::R regs[NV];

    while (todo) {
        // ---- the rows of this pass: the first row left and every later one of its request with its first seen key
        const int lead = __ffs(todo) - 1;
        unsigned grp = 0;
        int p_max = 0;
        const int lo = lo_r[lead];
#pragma unroll
        for (int r = 0; r < R; ++r)
            if ((todo >> r & 1u) && sq[r] == sq[lead] && lo_r[r] == lo) {
                grp |= 1u << r;
                p_max = pr[r] > p_max ? pr[r] : p_max;
            }
        todo &= ~grp;
        const int* bt = block_table + (long)sq[lead] * max_blocks;
        __syncthreads();                                     // (the pass before has left shared memory)
        for (int i = tid; i < R * Hq * L.rs_q; i += TALK_THREADS) {
            const int rh = i / L.rs_q, d = i - rh * L.rs_q, r = rh / Hq, h = rh - r * Hq;
            qs[i] = ((grp >> r & 1u) && d < Dk) ? Elem<TA>::load(q + ((row0 + r) * Hq + h) * Dc + d) : 0.f;
        }
        for (int i = tid; i < R * Hq; i += TALK_THREADS) { ml[2 * i] = -INFINITY; ml[2 * i + 1] = 0.f; }
        float4 acc[TALK_ROWS_ACC][R];
#pragma unroll
        for (int i = 0; i < TALK_ROWS_ACC; ++i)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[i][r] = make_float4(0.f, 0.f, 0.f, 0.f);

        int j0 = lo + 64 * split, par = 0;
        if (j0 <= p_max) {
            const int j = j0 + lane;
            if (wave == 0) koff[lane] = j <= p_max ? (long)bt[j / P] * page_stride + (long)(j % P) * Dc : -1L;
            __syncthreads();
            talk_fetch<TA, NV>(regs, item_k, cache, koff, 0, (Hkv < HGk ? Hkv : HGk) * 64, 6, 0, head_stride);
        }
        for (; j0 <= p_max; j0 += 64 * KS, par ^= 1) {
            const long* ko = koff + par * 64;
            long* kn = koff + (par ^ 1) * 64;
            const int jn = j0 + 64 * KS;
            const bool more = jn <= p_max;
            const int j = j0 + lane;
            if (wave == 0) kn[lane] = jn + lane <= p_max ? (long)bt[(jn + lane) / P] * page_stride + (long)((jn + lane) % P) * Dc : -1L;
            for (int s = 0; s < nS; ++s) {
                const bool is_v = s >= nK;
                const int g0 = is_v ? 0 : s * HGk;
                const int hg = is_v ? Hkv : (Hkv - g0 < HGk ? Hkv - g0 : HGk);
                const int k0 = is_v ? (s - nK) << kps_shift : 0;
                __syncthreads();
                if (is_v) talk_commit<TA, NV>(regs, item_v, stage, Hkv * KPS, L.ls_v);
                else talk_commit<TA, NV>(regs, item_k, stage, hg * 64, L.ls_k);
                if (s + 1 < nS) {
                    if (s + 1 >= nK) {
                        talk_fetch<TA, NV>(regs, item_v, cache + plane, ko, 0, Hkv * KPS, kps_shift, (s + 1 - nK) << kps_shift,
                                           head_stride);
                    } else {
                        const int n0 = (s + 1) * HGk;
                        talk_fetch<TA, NV>(regs, item_k, cache, ko, n0, (Hkv - n0 < HGk ? Hkv - n0 : HGk) * 64, 6, 0, head_stride);
                    }
                } else if (more) {
                    talk_fetch<TA, NV>(regs, item_k, cache, kn, 0, (Hkv < HGk ? Hkv : HGk) * 64, 6, 0, head_stride);
                }
                __syncthreads();
                if (!is_v) {
                    // ---- scores of R rows: a key's numbers are read once for the R dot products
                    for (int h = g0 * G + wave; h < (g0 + hg) * G; h += TALK_THREADS / 64) {
                        float bv[R];
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            const int n = pr[r] - j;
                            bv[r] = (bias && (grp >> r & 1u) && n >= 0) ? bias[(long)(n < bias_rows ? n : bias_rows - 1) * Hq + h] : 0.f;
                        }
                        const float4* kr = (const float4*)(stage + (long)((h / G - g0) * 64 + lane) * L.ls_k);
                        float dt[R];
#pragma unroll
                        for (int r = 0; r < R; ++r) dt[r] = 0.f;
#pragma unroll 2
                        for (int d = 0; d < vpr_k; ++d) {
                            const float4 b = kr[d];
#pragma unroll
                            for (int r = 0; r < R; ++r) {
                                const float4 a = *(const float4*)(qs + (r * Hq + h) * L.rs_q + d * 4);
                                dt[r] = fmaf(a.x, b.x, dt[r]); dt[r] = fmaf(a.y, b.y, dt[r]);
                                dt[r] = fmaf(a.z, b.z, dt[r]); dt[r] = fmaf(a.w, b.w, dt[r]);
                            }
                        }
#pragma unroll
                        for (int r = 0; r < R; ++r) sc[(r * Hq + h) * 64 + lane] = dt[r] * scale + bv[r];
                    }
                    if (s == nK - 1) {
                        __syncthreads();
                        // ---- the heads' scores mixed, then the tile joins each row's and head's running softmax
                        for (int rh = wave; rh < R * Hq; rh += TALK_THREADS / 64) {
                            const int r = rh / Hq, h = rh - r * Hq;
                            if (!(grp >> r & 1u) || j0 > pr[r]) {            // not a row of this pass, or none of its keys here
                                pm[rh * 64 + lane] = 0.f;
                                if (lane == 0) al[rh] = 1.f;
                                continue;
                            }
                            const bool seen = j <= pr[r];
                            float sv;
                            if (talk) {
                                sv = 0.f;
                                for (int g = 0; g < Hq; ++g) sv = fmaf(tk[h * Hq + g], sc[(r * Hq + g) * 64 + lane], sv);
                            } else {
                                sv = sc[rh * 64 + lane];
                            }
                            if (!seen) sv = -INFINITY;
                            const float m_old = ml[2 * rh], l_old = ml[2 * rh + 1];
                            const float m_new = fmaxf(m_old, wave_max(sv));  // finite: key j0 is seen by this row
                            const float a = expf(m_old - m_new);
                            const float pj = seen ? expf(sv - m_new) : 0.f;
                            const float l_new = l_old * a + wave_sum(pj);
                            pm[rh * 64 + lane] = pj;
                            if (lane == 0) { ml[2 * rh] = m_new; ml[2 * rh + 1] = l_new; al[rh] = a; }
                        }
                    }
                } else {
                    // ---- the stage's values: a value's numbers are read once for the R sums
#pragma unroll
                    for (int i = 0; i < TALK_ROWS_ACC; ++i) {
                        const int h = hd[i] >> 16;
                        if (h < Hq) {
                            const float* vs = stage + (long)(h / G) * KPS * L.ls_v + (hd[i] & 0xffff);
                            float4 a[R];
#pragma unroll
                            for (int r = 0; r < R; ++r) {
                                const float f = k0 == 0 ? al[r * Hq + h] : 1.f;
                                a[r] = make_float4(acc[i][r].x * f, acc[i][r].y * f, acc[i][r].z * f, acc[i][r].w * f);
                            }
                            for (int jj = 0; jj < KPS; jj += 4) {
                                float4 w[R];
#pragma unroll
                                for (int r = 0; r < R; ++r) w[r] = *(const float4*)(pm + (r * Hq + h) * 64 + k0 + jj);
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const float4 vv = *(const float4*)(vs + (long)(jj + e) * L.ls_v);
#pragma unroll
                                    for (int r = 0; r < R; ++r) {
                                        const float we = e == 0 ? w[r].x : (e == 1 ? w[r].y : (e == 2 ? w[r].z : w[r].w));
                                        a[r].x = fmaf(we, vv.x, a[r].x); a[r].y = fmaf(we, vv.y, a[r].y);
                                        a[r].z = fmaf(we, vv.z, a[r].z); a[r].w = fmaf(we, vv.w, a[r].w);
                                    }
                                }
                            }
#pragma unroll
                            for (int r = 0; r < R; ++r) acc[i][r] = a[r];
                        }
                    }
                }
            }
        }
        __syncthreads();
        // ---- the pass's rows leave their results
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!(grp >> r & 1u)) continue;
            const long t = row0 + r;
            if (KS == 1) {
#pragma unroll
                for (int i = 0; i < TALK_ROWS_ACC; ++i) {
                    const int h = hd[i] >> 16, d = hd[i] & 0xffff;
                    if (h < Hq) {
                        const float f = out_scale / ml[2 * (r * Hq + h) + 1];
                        const float a[4] = {acc[i][r].x, acc[i][r].y, acc[i][r].z, acc[i][r].w};
                        for (int e = 0; e < 4; ++e)
                            if (d + e < Dv) Elem<TA>::store(out + t * out_stride + h * Dv + d + e, a[e] * f);
                    }
                }
            } else {
                float* w = ws + (t * KS + split) * (2 * Hq + n_out);
                for (int i = tid; i < 2 * Hq; i += TALK_THREADS) w[i] = ml[2 * r * Hq + i];
#pragma unroll
                for (int i = 0; i < TALK_ROWS_ACC; ++i) {
                    const int h = hd[i] >> 16, d = hd[i] & 0xffff;
                    if (h < Hq) {
                        const float a[4] = {acc[i][r].x, acc[i][r].y, acc[i][r].z, acc[i][r].w};
                        for (int e = 0; e < 4; ++e)
                            if (d + e < Dv) w[2 * Hq + h * Dv + d + e] = a[e];
                    }
                }
            }
        }
    }
}

// grid (tokens): the splits' partial results weighed by exp(m_s - max m) and added in the order of the splits
template <typename TA>
__global__ __launch_bounds__(TALK_THREADS) void attention_talk_merge_kernel(
    const float* __restrict__ ws, TA* __restrict__ out, long out_stride, float out_scale,
    const int* __restrict__ tokens, int Hq, int Dv, int KS) {
    const long t = tokens ? tokens[blockIdx.x] : blockIdx.x;
    const int n_out = Hq * Dv, rec = 2 * Hq + n_out;
    const float* w = ws + (long)blockIdx.x * KS * rec;
    for (int o = threadIdx.x; o < n_out; o += TALK_THREADS) {
        const int h = o / Dv;
        float m = -INFINITY;
        for (int s = 0; s < KS; ++s) m = fmaxf(m, w[(long)s * rec + 2 * h]);
        float l = 0.f, a = 0.f;
        for (int s = 0; s < KS; ++s) {
            const float f = expf(w[(long)s * rec + 2 * h] - m);          // (a split without keys: exp(-inf) = 0)
            l = fmaf(w[(long)s * rec + 2 * h + 1], f, l);
            a = fmaf(w[(long)s * rec + 2 * Hq + o], f, a);
        }
        Elem<TA>::store(out + t * out_stride + o, a / l * out_scale);
    }
}

// Into how many blocks a token's key tiles are dealt: none while the tokens alone fill the machine, else a split for
// every 128 of the most keys a token can see (max_keys: the chunk or window; 0 if unbounded: no split).
extern "C" int qe_attention_talk_splits(int n_tokens, int max_keys) {
    if (n_tokens <= 0 || max_keys <= 128) return 1;
    int ks = (max_keys + 127) / 128;
    if (ks > TALK_MAX_SPLITS) ks = TALK_MAX_SPLITS;
    const int room = 1024 / n_tokens;
    if (ks > room) ks = room;
    return ks < 1 ? 1 : ks;
}

// q [T, Hq, Dc] (a head's first Dk numbers are read); out: row t at out + t * out_stride, Hq * Dv numbers,
// multiplied by out_scale; bias float32 [bias_rows, Hq] or null; talk float32 [Hq, Hq] or null; tokens: null for
// all T rows, else n_tokens row indices; window as for first_seen_key; splits from qe_attention_talk_splits with
// ws of n_tokens * splits * (2 Hq + Hq Dv) floats (null for one split).
extern "C" int qe_attention_talk(const void* q, void* out, long out_stride, float out_scale, const void* cache,
                                 const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                                 const int* tokens, int n_tokens, const float* bias, int bias_rows, const float* talk,
                                 int Hq, int Hkv, int Dk, int Dv, int Dc, int P, float scale, int window, int splits,
                                 float* ws, int dt_a, hipStream_t stream) {
    QE_REQUIRE(n_tokens >= 0 && Hq > 0 && Hkv > 0 && Dk > 0 && Dv > 0 && P > 0 && max_blocks > 0, "talking attention: bad sizes");
    QE_REQUIRE(Hq % Hkv == 0, "talking attention: %d query heads are no multiple of %d key/value heads", Hq, Hkv);
    QE_REQUIRE(Dc % 4 == 0 && Dc >= ((Dk + 3) & ~3) && Dc >= ((Dv + 3) & ~3),
               "talking attention: heads of %d and %d numbers in a cache of %d (a multiple of 4)", Dk, Dv, Dc);
    QE_REQUIRE((long)Hq * ((Dv + 3) / 4) <= TALK_THREADS * TALK_MAX_ACC && Hq < 32768,
               "talking attention: %d heads of %d values are more than %d outputs", Hq, Dv, 4 * TALK_THREADS * TALK_MAX_ACC);
    QE_REQUIRE(!bias || bias_rows > 0, "talking attention: a bias table without rows");
    QE_REQUIRE(out_stride >= (long)Hq * Dv, "talking attention: output rows overlap");
    QE_REQUIRE(splits >= 1 && splits <= TALK_MAX_SPLITS && (splits == 1 || ws), "talking attention: %d splits", splits);
    if (n_tokens == 0) return 0;
    const TalkLayout L0 = talk_layout(Hq, Hkv, Dk, Dv, 1, 4);
    const int vk = L0.rs_q >> 2, vv = L0.ls_v >> 2;
    QE_REQUIRE(vk <= 64, "talking attention: key heads of %d numbers (at most 256)", Dk);
    QE_REQUIRE((long)Hkv * 4 * vv <= TALK_THREADS * 16, "talking attention: %d value heads of %d numbers", Hkv, Dv);
    // pieces a thread holds of a stage (256 * nv pieces a stage)
    const int nv = (vk > 32 || (long)Hkv * 4 * vv > TALK_THREADS * 8) ? 16 : 8;
    int hgk = 4 * nv / vk;
    hgk = hgk > Hkv ? Hkv : hgk;
    int kps_shift = 6;                                      // keys of a stage of values: a power of two from 4 to 64
    while (kps_shift > 2 && ((long)Hkv << kps_shift) * vv > TALK_THREADS * nv) --kps_shift;
    const TalkLayout L = talk_layout(Hq, Hkv, Dk, Dv, hgk, 1 << kps_shift);
    const size_t shmem = (size_t)L.total * sizeof(float);
    QE_REQUIRE(shmem <= 150 * 1024, "talking attention: %zu bytes of shared memory", shmem);
    dim3 grid(n_tokens, splits);
    // many rows (portions of prompts): several neighbouring rows a block, where shared memory holds their scores
    const int R = TALK_ROWS;
    const TalkRowsLayout LR = talk_rows_layout(L, R, Hq);
    const size_t shmem_rows = (size_t)LR.total * sizeof(float);
    const bool rows = !tokens && n_tokens >= 64 && nv == 8 && shmem_rows <= 100 * 1024 &&
                      (long)Hq * vv <= TALK_THREADS * TALK_ROWS_ACC;
#define QE_TALK_ROWS(TA_)                                                                                            \
    do {                                                                                                             \
        if (shmem_rows > 48 * 1024)                                                                                  \
            (void)hipFuncSetAttribute((const void*)attention_talk_rows_kernel<TA_, 8, TALK_ROWS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem_rows); \
        attention_talk_rows_kernel<TA_, 8, TALK_ROWS><<<dim3((n_tokens + R - 1) / R, splits), TALK_THREADS, shmem_rows, stream>>>( \
            (const TA_*)q, (TA_*)out, out_stride, out_scale, (const TA_*)cache, positions, tok_seq, block_table,     \
            max_blocks, n_tokens, bias, bias_rows, talk, Hq, Hkv, Dk, Dv, Dc, P, scale, window, splits, hgk, kps_shift, ws); \
        if (splits > 1)                                                                                              \
            attention_talk_merge_kernel<TA_><<<n_tokens, TALK_THREADS, 0, stream>>>(ws, (TA_*)out, out_stride,       \
                                                                                    out_scale, tokens, Hq, Dv, splits); \
    } while (0)
#define QE_TALK2(TA_, NV_)                                                                                           \
    do {                                                                                                             \
        if (shmem > 48 * 1024)                                                                                       \
            (void)hipFuncSetAttribute((const void*)attention_talk_kernel<TA_, NV_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem); \
        attention_talk_kernel<TA_, NV_><<<grid, TALK_THREADS, shmem, stream>>>(                                      \
            (const TA_*)q, (TA_*)out, out_stride, out_scale, (const TA_*)cache, positions, tok_seq, block_table,     \
            max_blocks, tokens, bias, bias_rows, talk, Hq, Hkv, Dk, Dv, Dc, P, scale, window, splits, hgk, kps_shift, ws); \
        if (splits > 1)                                                                                              \
            attention_talk_merge_kernel<TA_><<<n_tokens, TALK_THREADS, 0, stream>>>(ws, (TA_*)out, out_stride,       \
                                                                                    out_scale, tokens, Hq, Dv, splits); \
    } while (0)
#define QE_TALK(TA_) do { if (rows) QE_TALK_ROWS(TA_); else if (nv == 8) QE_TALK2(TA_, 8); else QE_TALK2(TA_, 16); } while (0)
    if (dt_a == QE_F32) QE_TALK(float);
    else if (dt_a == QE_BF16) QE_TALK(bf16_t);
    else QE_REQUIRE(false, "talking attention: unknown element type %d", dt_a);
#undef QE_TALK
#undef QE_TALK2
#undef QE_TALK_ROWS
    QE_LAUNCH_CHECK();
    return 0;
}
