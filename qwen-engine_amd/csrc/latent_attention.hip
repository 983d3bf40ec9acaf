// Attention over one cached latent per token.
//
// A token's cache entry is one row [R + Dr]: the normed latent c (R numbers), from which every head's
// keys and values are linear maps (k_h = Uk_h c, v_h = Uv_h c), and one rotated key part (Dr numbers)
// that all heads share.  With the key map folded into the query (q'_h = Uk_h^T q_h) a head's score
// against a token is q'_h . c + q_rot_h . k_rot: one dot product of R + Dr numbers against the
// cached row, and the head's output in latent space is sum_j p_j c_j, which Uv_h then maps to the
// head's values.  So all heads read the same rows: one key/value "head" of size R + Dr whose first R
// numbers are also the value.
//
// cache of one layer: [page][P][R + Dr]; slot = page * P + offset addresses a row.
//
//   qe_latent_kv_store   the projection's row [R + Dr] (32-bit) -> c = w * u / rms(u) over the first
//                        R, the interleaved rotation over the last Dr by the token's position, into the
//                        cache row of the token's slot (negative: nowhere)
//   qe_latent_q_rotate   the rotated parts of the queries into the packed queries [T, H, R + Dr]
//   qe_latent_attention  softmax(scale * q . rows) . rows[:R] per (token, head) over the request's
//                        positions 0 .. p, 32-bit throughout, any sizes
//
// The rotation turns the pair (2i, 2i + 1), i < dims / 2, by position * inv_freq[i], or, half-split, the pair
// (i, i + dims / 2); the angle, its sine and cosine are 32-bit.
//
// A window of W keys (a token at position p sees the positions p - W + 1 .. p) and a sink (one number a head that
// joins the softmax's denominator and carries no value) are parameters of the attention kernels.
#include "common.h"

#define LAT_MAX_R 2048

__device__ __forceinline__ void turn_pair(float angle, float& u, float& v) {
    float s, c;
    sincosf(angle, &s, &c);
    const float a = u * c - v * s, b = v * c + u * s;
    u = a;
    v = b;
}

// Item i of ceil(Dr / 2) handles the numbers a and b (b may lie beyond Dr) and turns them or not.
__device__ __forceinline__ void pair_place(int i, int rot_dims, int half_split, int& a, int& b, bool& turn) {
    const int hr = rot_dims >> 1;
    if (half_split && i < hr) {
        a = i;
        b = i + hr;
        turn = true;
    } else {
        a = 2 * i;
        b = 2 * i + 1;
        turn = !half_split && b < rot_dims;
    }
}

// q (may be null) [T, H, Dn + Dr] -> qp [T, H, R + Dr]: in the same launch, the rotated parts of the token's
// queries go to the packed queries (what qe_latent_q_rotate does), so that a step of few rows has a kernel less.
template <typename TC>
__global__ void latent_kv_store_kernel(const float* __restrict__ kv, const float* __restrict__ weight, float eps,
                                       const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                       int rot_dims, const int* __restrict__ slots, TC* __restrict__ cache,
                                       int R, int Dr, const TC* __restrict__ q, TC* __restrict__ qp, int H, int Dn,
                                       int half_split) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    if (q) {
        const float pq = (float)positions[t];
        const int pairs = (Dr + 1) / 2;
        for (int idx = threadIdx.x; idx < H * pairs; idx += blockDim.x) {
            const int h = idx / pairs, i = idx % pairs;
            const TC* src = q + (t * H + h) * (Dn + Dr) + Dn;
            TC* dst = qp + (t * H + h) * (R + Dr) + R;
            int a, b;
            bool turn;
            pair_place(i, rot_dims, half_split, a, b, turn);
            if (b >= Dr) {
                Elem<TC>::store(dst + a, Elem<TC>::load(src + a));
                continue;
            }
            float u = Elem<TC>::load(src + a), v = Elem<TC>::load(src + b);
            if (turn) turn_pair(pq * inv_freq[i], u, v);
            Elem<TC>::store(dst + a, u);
            Elem<TC>::store(dst + b, v);
        }
    }
    const float* row = kv + t * (R + Dr);
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += blockDim.x) ss += row[i] * row[i];
    ss = block_sum(ss, red);
    const int slot = slots ? slots[t] : -1;
    if (slot < 0) return;
    const float f = rsqrtf(ss / (float)R + eps);
    TC* dst = cache + (long)slot * (R + Dr);
    for (int i = threadIdx.x; i < R; i += blockDim.x) Elem<TC>::store(dst + i, row[i] * f * weight[i]);
    const float p = (float)positions[t];
    for (int i = threadIdx.x; i < (Dr + 1) / 2; i += blockDim.x) {
        int a, b;
        bool turn;
        pair_place(i, rot_dims, half_split, a, b, turn);
        if (b >= Dr) {                                                 // an odd last number passes
            Elem<TC>::store(dst + R + a, row[R + a]);
            continue;
        }
        float u = row[R + a], v = row[R + b];
        if (turn) turn_pair(p * inv_freq[i], u, v);
        Elem<TC>::store(dst + R + a, u);
        Elem<TC>::store(dst + R + b, v);
    }
}

extern "C" int qe_latent_kv_store(const float* kv, const float* weight, float eps, const int* positions,
                                  const float* inv_freq, int rot_dims, const int* slots, void* cache, int dt_c,
                                  int T, int R, int Dr, const void* q, void* qp, int H, int Dn, int half_split,
                                  hipStream_t stream) {
    QE_REQUIRE(!q || (qp && H > 0 && Dn >= 0), "latent_kv_store: queries without a place for them");
    QE_REQUIRE(T >= 0 && R > 0 && Dr >= 0, "latent_kv_store: bad sizes T=%d R=%d Dr=%d", T, R, Dr);
    QE_REQUIRE(rot_dims >= 0 && rot_dims <= Dr && rot_dims % 2 == 0, "latent_kv_store: %d rotated of %d", rot_dims, Dr);
    if (T == 0) return 0;
    const int threads = R >= 512 ? 256 : 64;
    if (dt_c == QE_F32)
        latent_kv_store_kernel<float><<<T, threads, 0, stream>>>(kv, weight, eps, positions, inv_freq, rot_dims, slots,
                                                                  (float*)cache, R, Dr, (const float*)q, (float*)qp, H, Dn, half_split);
    else if (dt_c == QE_BF16)
        latent_kv_store_kernel<bf16_t><<<T, threads, 0, stream>>>(kv, weight, eps, positions, inv_freq, rot_dims, slots,
                                                                   (bf16_t*)cache, R, Dr, (const bf16_t*)q, (bf16_t*)qp, H, Dn, half_split);
    else
        QE_REQUIRE(false, "latent_kv_store: unknown cache type %d", dt_c);
    QE_LAUNCH_CHECK();
    return 0;
}

// q [T, H, Dn + Dr] -> qp[T, H, R + Dr]: the last Dr of each head, rotated, to the last Dr of the
// packed query (its first R come from the product with the folded key map).
template <typename TA>
__global__ void latent_q_rotate_kernel(const TA* __restrict__ q, const int* __restrict__ positions,
                                       const float* __restrict__ inv_freq, int rot_dims, TA* __restrict__ qp,
                                       long n_heads_total, int H, int Dn, int Dr, int R, int half_split) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;      // (token * H + head) * ceil(Dr / 2) + pair
    const int pairs = (Dr + 1) / 2;
    if (idx >= n_heads_total * pairs) return;
    const long th = idx / pairs;
    const int i = (int)(idx % pairs);
    const long t = th / H;
    const TA* src = q + th * (Dn + Dr) + Dn;
    TA* dst = qp + th * (R + Dr) + R;
    int a, b;
    bool turn;
    pair_place(i, rot_dims, half_split, a, b, turn);
    if (b >= Dr) {                                                     // an odd last number passes
        Elem<TA>::store(dst + a, Elem<TA>::load(src + a));
        return;
    }
    float u = Elem<TA>::load(src + a), v = Elem<TA>::load(src + b);
    if (turn) turn_pair((float)positions[t] * inv_freq[i], u, v);
    Elem<TA>::store(dst + a, u);
    Elem<TA>::store(dst + b, v);
}

extern "C" int qe_latent_q_rotate(const void* q, const int* positions, const float* inv_freq, int rot_dims, void* qp,
                                  int dt_a, int T, int H, int Dn, int Dr, int R, int half_split, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && Dn >= 0 && Dr >= 0 && R > 0, "latent_q_rotate: bad sizes");
    QE_REQUIRE(rot_dims >= 0 && rot_dims <= Dr && rot_dims % 2 == 0, "latent_q_rotate: %d rotated of %d", rot_dims, Dr);
    const long n = (long)T * H * ((Dr + 1) / 2);
    if (n == 0) return 0;
    const int blocks = qe_cdiv(n, 256);
    if (dt_a == QE_F32)
        latent_q_rotate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)q, positions, inv_freq, rot_dims,
                                                                   (float*)qp, (long)T * H, H, Dn, Dr, R, half_split);
    else if (dt_a == QE_BF16)
        latent_q_rotate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)q, positions, inv_freq, rot_dims,
                                                                    (bf16_t*)qp, (long)T * H, H, Dn, Dr, R, half_split);
    else
        QE_REQUIRE(false, "latent_q_rotate: unknown type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// One wave per (token, head).  Keys are taken 64 at a time from the first position the token sees (0, or
// p - window + 1) upwards with an online softmax, so the order of the sums depends on the position only: not on
// how the request's tokens were cut into steps, nor on what else is in the batch.  The sink joins at the end.
template <typename TA>
__global__ __launch_bounds__(64) void latent_attention_kernel(
    const TA* __restrict__ qp, TA* __restrict__ out, const TA* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int H, int R, int Dr, int P, float scale, int window, const float* __restrict__ sink) {
    extern __shared__ float smem[];
    const int D = R + Dr;
    float* qs = smem;                                   // D
    float* ps = smem + D;                               // 64 weights of the current chunk
    long* roff = (long*)(smem + ((D + 64 + 1) & ~1));   // 64 offsets of the chunk's rows
    const long t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int p = positions[t];
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const TA* qrow = qp + (t * H + h) * D;
    for (int d = lane; d < D; d += 64) qs[d] = Elem<TA>::load(qrow + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[LAT_MAX_R / 64];
#pragma unroll
    for (int i = 0; i < LAT_MAX_R / 64; ++i) acc[i] = 0.f;

    const int first = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    for (int j0 = first; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float sc = -INFINITY;
        long ro = 0;
        if (j <= p) {
            ro = ((long)bt[j / P] * P + j % P) * D;
            const TA* krow = cache + ro;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], Elem<TA>::load(krow + d), dot);
            sc = dot * scale;
        }
        const float mn = fmaxf(m, wave_max(sc));
        const float alpha = expf(m - mn);
        const float pj = (j <= p) ? expf(sc - mn) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = mn;
        ps[lane] = pj;
        roff[lane] = ro;
        __syncthreads();
        const int cnt = (p - j0 + 1 < 64) ? p - j0 + 1 : 64;
#pragma unroll
        for (int i = 0; i < LAT_MAX_R / 64; ++i) {
            const int d = lane + i * 64;
            if (d < R) {
                float a = acc[i] * alpha;
                for (int jj = 0; jj < cnt; ++jj) a = fmaf(ps[jj], Elem<TA>::load(cache + roff[jj] + d), a);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
    float inv = 1.f / l;
    if (sink) {                                        // one more entry of score sink[h], with no value
        const float sk = sink[h], mt = fmaxf(m, sk), f = expf(m - mt);
        inv = f / (l * f + expf(sk - mt));
    }
    TA* orow = out + (t * H + h) * R;
#pragma unroll
    for (int i = 0; i < LAT_MAX_R / 64; ++i) {
        const int d = lane + i * 64;
        if (d < R) Elem<TA>::store(orow + d, acc[i] * inv);
    }
}

// qp [T, H, R + Dr] -> out [T, H, R]
extern "C" int qe_latent_attention(const void* qp, void* out, const void* cache, const int* positions,
                                   const int* tok_seq, const int* block_table, int max_blocks, int T, int H, int R,
                                   int Dr, int P, float scale, int window, const float* sink, int dt_a,
                                   hipStream_t stream) {
    QE_REQUIRE(window >= 0, "latent_attention: a window of %d keys", window);
    QE_REQUIRE(R > 0 && R <= LAT_MAX_R, "latent_attention: latent size %d exceeds %d", R, LAT_MAX_R);
    QE_REQUIRE(H > 0 && H <= 65535 && Dr >= 0 && P > 0, "latent_attention: bad sizes");
    if (T == 0) return 0;
    dim3 grid(T, H);
    const size_t shmem = (size_t)((R + Dr + 64 + 1) & ~1) * sizeof(float) + 64 * sizeof(long);
    if (dt_a == QE_F32)
        latent_attention_kernel<float><<<grid, 64, shmem, stream>>>((const float*)qp, (float*)out, (const float*)cache,
                                                                     positions, tok_seq, block_table, max_blocks, H, R, Dr, P, scale, window, sink);
    else if (dt_a == QE_BF16)
        latent_attention_kernel<bf16_t><<<grid, 64, shmem, stream>>>((const bf16_t*)qp, (bf16_t*)out, (const bf16_t*)cache,
                                                                      positions, tok_seq, block_table, max_blocks, H, R, Dr, P, scale, window, sink);
    else
        QE_REQUIRE(false, "latent_attention: unknown type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}
