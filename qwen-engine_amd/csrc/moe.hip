// Mixture of experts: routing, grouping of the (token, choice) pairs by expert, and the experts'
// two matrix products over the grouped rows.  Everything happens on the device, with grids that depend
// on the shapes only (a block that finds no tile for itself leaves), so a step can be recorded.
//
//   qe_moe_route   scores = softmax(logits) over all experts (32-bit).  The experts form G equal groups
//                  of neighbours; a group's score is its largest; only the experts of the ``keep`` best
//                  groups can be chosen; of those the ``top`` largest are, weighted by their scores as
//                  they are.  On ties the lower index wins.  ids [T, top], weights [T, top].
//   qe_moe_route_biased  scores = softmax(logits) over all experts (32-bit); the ``top`` largest of
//                  score + correction are chosen (on ties the lower index), weighted by their scores
//                  without the correction, divided by the chosen scores' sum (+ 1e-20), times ``scale``.
//   qe_moe_identity  the experts from E_real on are the identity: a pair that chose one contributes its
//                  token's row itself; they get no tiles from qe_moe_sort (tile_experts).
//   qe_moe_sort    perm [T * top]: the pairs (as index t * top + j) ordered by expert; tiles
//                  [max_tiles, 3] = (expert, first sorted row, rows <= tile_rows) and their number.
//   qe_moe_gather  xs[i] = x[perm[i] / top]: the pairs' rows side by side, for a product that wants its rows
//                  contiguous; qe_moe_combine  out[t] = sum_j weights[t, j] y[inv[t top + j]] in the order of j
//                  (32-bit): the way back.
//   qe_moe_gemm    for every tile, rows . W_e^T:
//                    first product  (dual): x row of the pair's token against gate and up rows of
//                      W_e [2 F, K]; g = min(g, limit), u = clamp(u, -limit, limit),
//                      a = g sigmoid(slope g) (u + 1), stored at the sorted row
//                    second product (weighted): a's sorted row against W_e [N, K], times the pair's
//                      weight, to parts[j][t] (32-bit): the norm that follows adds a token's ``top``
//                      parts in the order of j.
//                    dual == 2: one matrix W_e [F, K] and a = relu(W_e x)^2 instead.
//                  Any sizes, every multiply-add in IEEE 32-bit.
#include "common.h"

__device__ __forceinline__ void wave_argmax(float& v, int& i) {
    for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        if (ov > v || (ov == v && oi >= 0 && (i < 0 || oi < i))) { v = ov; i = oi; }
    }
}

// One wave per token.  Marks in the score table: -2 not (or no longer) a candidate.
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, int* __restrict__ ids,
                                                       float* __restrict__ weights, int E, int G, int keep, int top) {
    extern __shared__ float sc[];          // E scores, G group scores
    float* gs = sc + E;
    const long t = blockIdx.x;
    const int lane = threadIdx.x;
    const float* z = logits + t * E;
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
        const float ex = expf(z[e] - mx);
        sc[e] = ex;
        sum += ex;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) {
        float v = sc[e] / sum;
        if (!(v == v)) v = 0.f;            // (a row of garbage still gets experts inside the table)
        sc[e] = v;
    }
    __syncthreads();
    if (keep < G) {
        const int per = E / G;
        for (int g = lane; g < G; g += 64) {
            float m = -1.f;
            for (int e = g * per; e < (g + 1) * per; ++e) m = fmaxf(m, sc[e]);
            gs[g] = m;
        }
        __syncthreads();
        for (int r = 0; r < keep; ++r) {
            float bv = -1.f;
            int bi = -1;
            for (int g = lane; g < G; g += 64)
                if (gs[g] > bv) { bv = gs[g]; bi = g; }
            wave_argmax(bv, bi);
            if (lane == 0 && bi >= 0) gs[bi] = -3.f;       // kept
            __syncthreads();
        }
        for (int e = lane; e < E; e += 64)
            if (gs[e / per] != -3.f) sc[e] = -2.f;
        __syncthreads();
    }
    for (int r = 0; r < top; ++r) {
        float bv = -1.f;
        int bi = -1;
        for (int e = lane; e < E; e += 64)
            if (sc[e] > bv) { bv = sc[e]; bi = e; }
        wave_argmax(bv, bi);
        if (lane == 0) {
            ids[t * top + r] = bi >= 0 ? bi : 0;
            weights[t * top + r] = bi >= 0 ? bv : 0.f;
            if (bi >= 0) sc[bi] = -2.f;
        }
        __syncthreads();
    }
}

extern "C" int qe_moe_route(const float* logits, int* ids, float* weights, int T, int E, int G, int keep, int top,
                            hipStream_t stream) {
    QE_REQUIRE(T >= 0 && E > 0 && G > 0 && E % G == 0, "moe_route: %d experts in %d groups", E, G);
    QE_REQUIRE(keep >= 1 && keep <= G && top >= 1 && top <= keep * (E / G), "moe_route: top %d of %d groups of %d", top, keep, E / G);
    QE_REQUIRE((E + G) * sizeof(float) <= 60000, "moe_route: too many experts");
    if (T == 0) return 0;
    moe_route_kernel<<<T, 64, (E + G) * sizeof(float), stream>>>(logits, ids, weights, E, G, keep, top);
    QE_LAUNCH_CHECK();
    return 0;
}


// One token's routing by one wave: softmax over all E outputs, choice by score + correction, weights from the
// scores alone.  Without a correction (null) the choice goes by the logits themselves and the weights are the
// softmax over the chosen logits alone (the scores stay unnormalised: the largest is 1, so the chosen ones' sum
// is at least 1 however far the others lie below).  sc: the wave's own 2 E + top floats of shared memory.  Every wave of the block calls it together
// (the barriers are the block's); a wave without a token (z null) only keeps step.
__device__ __forceinline__ void route_biased_token(const float* __restrict__ z, const float* __restrict__ correction,
                                                   float* sc, int* __restrict__ ids, float* __restrict__ weights, int E,
                                                   int top, float scale, int lane, long zs = 1,
                                                   const float* __restrict__ zbias = nullptr) {
    float* ch = sc + E;
    float* picked = ch + E;
    if (z) {                                             // (zs: the distance between a token's logits; zbias: added to them)
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) {
            const float zv = z[e * zs] + (zbias ? zbias[e] : 0.f);
            ch[e] = zv;
            mx = fmaxf(mx, zv);
        }
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float ex = expf(ch[e] - mx);
            sc[e] = ex;
            sum += ex;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += 64) {
            float v = correction ? sc[e] / sum : sc[e];
            if (!(v == v)) v = 0.f;            // (a row of garbage still gets experts inside the table)
            sc[e] = v;
            float c = correction ? v + correction[e] : ch[e];
            if (!(c == c)) c = correction ? 0.f : -3.0e38f;
            ch[e] = c;
        }
    }
    __syncthreads();
    for (int r = 0; r < top; ++r) {
        if (z) {
            float bv = -INFINITY;
            int bi = -1;
            for (int e = lane; e < E; e += 64)
                if (ch[e] > bv) { bv = ch[e]; bi = e; }
            wave_argmax(bv, bi);
            if (lane == 0) {
                ids[r] = bi >= 0 ? bi : 0;
                picked[r] = bi >= 0 ? sc[bi] : 0.f;
                if (bi >= 0) ch[bi] = -INFINITY;
            }
        }
        __syncthreads();
    }
    if (z && lane == 0) {
        float tot = 0.f;
        for (int r = 0; r < top; ++r) tot += picked[r];
        for (int r = 0; r < top; ++r) weights[r] = picked[r] / (tot + 1e-20f) * scale;
    }
}

__global__ __launch_bounds__(64) void moe_route_biased_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                                              int* __restrict__ ids, float* __restrict__ weights, int E, int top,
                                                              float scale, int transposed, const float* __restrict__ zbias,
                                                              int ld) {
    extern __shared__ float sc[];          // E scores, E choice scores, top chosen scores
    const long t = blockIdx.x;
    // (transposed: logits [E, T], as a product of the router's few rows against the tokens' many leaves them)
    route_biased_token(transposed ? logits + t : logits + t * ld, correction, sc, ids + t * top, weights + t * top, E, top,
                       scale, threadIdx.x, transposed ? (long)gridDim.x : 1L, zbias);
}

extern "C" int qe_moe_route_biased(const float* logits, const float* correction, int* ids, float* weights, int T, int E,
                                   int top, float scale, int transposed, const float* zbias, int ld, hipStream_t stream) {
    if (ld <= 0) ld = E;                   // (ld: the distance between two tokens' logits where they are not transposed)
    QE_REQUIRE(ld >= E, "moe_route_biased: rows of %d logits for %d experts", ld, E);
    QE_REQUIRE(T >= 0 && E > 0 && top >= 1 && top <= E, "moe_route_biased: top %d of %d experts", top, E);
    QE_REQUIRE((2 * E + top) * sizeof(float) <= 60000, "moe_route_biased: too many experts");
    if (T == 0) return 0;
    moe_route_biased_kernel<<<T, 64, (2 * E + top) * sizeof(float), stream>>>(logits, correction, ids, weights, E, top, scale, transposed, zbias, ld);
    QE_LAUNCH_CHECK();
    return 0;
}

// One block per (token, choice) pair that chose an identity expert (id >= E_real): its part of the output is the
// token's row itself.  parts != null: parts[j][t] = weight * x[t] (32-bit); else y[inv[pair]] = x[t] (32-bit), for a
// caller that weighs and adds the sorted rows afterwards.
template <typename TA, typename TY>
__global__ void moe_identity_kernel(const TA* __restrict__ x, const int* __restrict__ ids, const float* __restrict__ weights,
                                    const int* __restrict__ inv, float* __restrict__ parts, TY* __restrict__ y,
                                    int T, int top, int H, int E_real) {
    const long pair = blockIdx.x;
    if (ids[pair] < E_real) return;
    const long t = pair / top;
    const int j = pair % top;
    const TA* src = x + t * H;
    if (parts) {
        const float wgt = weights[pair];
        float* dst = parts + ((long)j * T + t) * H;
        for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = wgt * Elem<TA>::load(src + c);
    } else {
        TY* dst = y + (long)inv[pair] * H;
        for (int c = threadIdx.x; c < H; c += blockDim.x) Elem<TY>::store(dst + c, Elem<TA>::load(src + c));
    }
}

// y: sorted rows in x's type if y_as_x, else float
extern "C" int qe_moe_identity(const void* x, const int* ids, const float* weights, const int* inv, float* parts, void* y,
                               int T, int top, int H, int E_real, int dt_a, int y_as_x, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && top > 0 && H > 0 && E_real >= 0, "moe_identity: bad sizes");
    QE_REQUIRE((parts != nullptr) != (y != nullptr), "moe_identity: parts or sorted rows, one of them");
    QE_REQUIRE(parts || inv, "moe_identity: sorted rows need the pairs' places");
    if (T == 0) return 0;
    if (dt_a == QE_BF16 && y_as_x) moe_identity_kernel<bf16_t, bf16_t><<<T * top, 256, 0, stream>>>((const bf16_t*)x, ids, weights, inv, parts, (bf16_t*)y, T, top, H, E_real);
    else if (dt_a == QE_BF16) moe_identity_kernel<bf16_t, float><<<T * top, 256, 0, stream>>>((const bf16_t*)x, ids, weights, inv, parts, (float*)y, T, top, H, E_real);
    else if (dt_a == QE_F32) moe_identity_kernel<float, float><<<T * top, 256, 0, stream>>>((const float*)x, ids, weights, inv, parts, (float*)y, T, top, H, E_real);
    else QE_REQUIRE(false, "moe_identity: unknown type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// One block.  n = T * top pairs.  Only the first tile_experts experts get tiles (the others' pairs still get
// their places in perm, behind them).
__device__ __forceinline__ void sort_pairs(const int* ids, int n, int E, int tile_experts, int tile_rows,
                                           int* __restrict__ perm, int* __restrict__ inv, int* __restrict__ tiles,
                                           int* __restrict__ n_tiles, int* counts, int* cursor) {
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) counts[e] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += blockDim.x) atomicAdd(&counts[ids[i]], 1);
    __syncthreads();
    for (int e = tid; e < E; e += blockDim.x) {
        int off = 0, tb = 0;
        for (int j = 0; j < e; ++j) {
            off += counts[j];
            if (j < tile_experts) tb += (counts[j] + tile_rows - 1) / tile_rows;
        }
        cursor[e] = off;
        const int c = counts[e];
        const int mine = e < tile_experts ? (c + tile_rows - 1) / tile_rows : 0;
        for (int k = 0; k < mine; ++k) {
            tiles[3 * (tb + k)] = e;
            tiles[3 * (tb + k) + 1] = off + k * tile_rows;
            tiles[3 * (tb + k) + 2] = c - k * tile_rows < tile_rows ? c - k * tile_rows : tile_rows;
        }
        if (e == tile_experts - 1) n_tiles[0] = tb + mine;
    }
    __syncthreads();
    for (int i = tid; i < n; i += blockDim.x) {
        const int at = atomicAdd(&cursor[ids[i]], 1);
        perm[at] = i;
        if (inv) inv[i] = at;
    }
}

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int n, int E, int tile_experts, int tile_rows,
                                                        int* __restrict__ perm, int* __restrict__ inv,
                                                        int* __restrict__ tiles, int* __restrict__ n_tiles) {
    extern __shared__ int sm[];
    sort_pairs(ids, n, E, tile_experts, tile_rows, perm, inv, tiles, n_tiles, sm, sm + E);
}

// A step of few tokens (T * top <= 1024 pairs): routing, sort and the identity experts' rows in one launch of one
// block, where three launches cost three times a dependent kernel's few microseconds.  Wave w routes the tokens
// w, w + 16, ...; the pairs' ids stay in shared memory for the sort; then every pair that chose an identity expert
// gets its token's row, weighted, as its part.
template <typename TA>
__global__ __launch_bounds__(1024) void moe_front_small_kernel(
    const float* __restrict__ logits, const float* __restrict__ correction, const TA* __restrict__ x, int* __restrict__ ids,
    float* __restrict__ weights, int* __restrict__ perm, int* __restrict__ inv, int* __restrict__ tiles,
    int* __restrict__ n_tiles, float* __restrict__ parts, int T, int H, int E, int E_real, int top, float scale, int tile_rows,
    const float* __restrict__ zbias, int ld) {
    extern __shared__ int sm[];
    const int n = T * top;
    int* ids_s = sm;                                     // n
    float* w_s = (float*)(sm + n);                       // n
    int* counts = sm + 2 * n;                            // E, then E cursors
    float* wave_sc = (float*)(sm + 2 * n + 2 * E);       // 16 waves of 2 E + top
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    for (int t0 = 0; t0 < T; t0 += waves) {
        const int t = t0 + wave;
        route_biased_token(t < T ? logits + (long)t * ld : nullptr, correction, wave_sc + (long)wave * (2 * E + top),
                           ids_s + (t < T ? t : 0) * top, w_s + (t < T ? t : 0) * top, E, top, scale, lane, 1L, zbias);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        ids[i] = ids_s[i];
        weights[i] = w_s[i];
    }
    sort_pairs(ids_s, n, E, E_real, tile_rows, perm, inv, tiles, n_tiles, counts, counts + E);
    if (E_real < E) {
        for (int i = 0; i < n; ++i) {
            if (ids_s[i] < E_real) continue;
            const int t = i / top, j = i - t * top;
            const float wgt = w_s[i];
            float* dst = parts + ((long)j * T + t) * H;
            const TA* src = x + (long)t * H;
            for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = wgt * Elem<TA>::load(src + c);
        }
    }
}

extern "C" int qe_moe_front_small_supported(int T, int E, int top) {
    return T > 0 && (long)T * top <= 1024 && ((long)2 * T * top + 2 * E + 16L * (2 * E + top)) * 4 <= 60000;
}

// logits float [T, E] (experts and identity experts together), correction [E]; ids, weights [T, top]; perm, inv
// [T top]; tiles, n_tiles as qe_moe_sort leaves them for the first E_real experts; parts float [top, T, H]: the
// parts of the pairs that chose an identity expert (E_real .. E - 1) are written, the others left.
extern "C" int qe_moe_front_small(const float* logits, const float* correction, const void* x, int* ids, float* weights,
                                  int* perm, int* inv, int* tiles, int* n_tiles, float* parts, int max_tiles, int T, int H,
                                  int E, int E_real, int top, float scale, int tile_rows, int dt_a, const float* zbias, int ld,
                                  hipStream_t stream) {
    if (ld <= 0) ld = E;
    QE_REQUIRE(qe_moe_front_small_supported(T, E, top), "moe_front_small: %d tokens, %d outputs, top %d", T, E, top);
    QE_REQUIRE(E_real >= 1 && E_real <= E && top <= E && tile_rows > 0 && H > 0, "moe_front_small: bad sizes");
    const int n = T * top;
    QE_REQUIRE(max_tiles >= (n + tile_rows - 1) / tile_rows + (E_real < n ? E_real : n), "moe_front_small: %d tiles may not be enough", max_tiles);
    const size_t lds = ((size_t)2 * n + 2 * E + 16 * (2 * E + top)) * 4;
    if (dt_a == QE_BF16)
        moe_front_small_kernel<bf16_t><<<1, 1024, lds, stream>>>(logits, correction, (const bf16_t*)x, ids, weights, perm, inv, tiles, n_tiles, parts, T, H, E, E_real, top, scale, tile_rows, zbias, ld);
    else if (dt_a == QE_F32)
        moe_front_small_kernel<float><<<1, 1024, lds, stream>>>(logits, correction, (const float*)x, ids, weights, perm, inv, tiles, n_tiles, parts, T, H, E, E_real, top, scale, tile_rows, zbias, ld);
    else
        QE_REQUIRE(false, "moe_front_small: unknown type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// inv (may be null): the sorted row of every pair, perm's inverse
extern "C" int qe_moe_sort(const int* ids, int n, int E, int tile_experts, int tile_rows, int* perm, int* inv, int* tiles,
                           int* n_tiles, int max_tiles, hipStream_t stream) {
    QE_REQUIRE(n >= 0 && E > 0 && tile_rows > 0 && tile_experts >= 1 && tile_experts <= E, "moe_sort: bad sizes");
    QE_REQUIRE(max_tiles >= (n + tile_rows - 1) / tile_rows + (tile_experts < n ? tile_experts : n), "moe_sort: %d tiles may not be enough", max_tiles);
    QE_REQUIRE(2 * E * sizeof(int) <= 60000, "moe_sort: too many experts");
    moe_sort_kernel<<<1, 1024, 2 * E * sizeof(int), stream>>>(ids, n, E, tile_experts, tile_rows, perm, inv, tiles, n_tiles);
    QE_LAUNCH_CHECK();
    return 0;
}

#define MT 64
#define MK 16

template <typename TA, typename TW, int MODE>      // 0: second product, weighted; 1: gate and up; 2: one matrix, squared relu
__global__ __launch_bounds__(256) void moe_gemm_kernel(
    const TA* __restrict__ x, const int* __restrict__ perm, int top, const TW* __restrict__ w, void* __restrict__ out_,
    const float* __restrict__ weights, const int* __restrict__ tiles, const int* __restrict__ n_tiles, int T, int N,
    int K, float limit, float slope, int interleaved) {
    constexpr bool DUAL = MODE == 1, FIRST = MODE != 0;
    if ((int)blockIdx.y >= n_tiles[0]) return;
    __shared__ float xs[MK][MT + 4];
    __shared__ float ws[MK][MT + 4];
    __shared__ float wu[DUAL ? MK : 1][MT + 4];
    __shared__ int src[MT];              // the row of x behind each row of the tile, -1 beyond its rows
    const int tid = threadIdx.x;
    const int e = tiles[3 * blockIdx.y], r0 = tiles[3 * blockIdx.y + 1], rows = tiles[3 * blockIdx.y + 2];
    const int n0 = blockIdx.x * MT;
    if (tid < MT) src[tid] = tid < rows ? (FIRST ? perm[r0 + tid] / top : r0 + tid) : -1;
    __syncthreads();
    const int lr = tid >> 2;
    const int lk = (tid & 3) * 4;
    const int ty = tid >> 4, tx = tid & 15;
    const TW* we = w + (long)e * (DUAL ? 2 : 1) * N * K;
    const int xrow = src[lr];
    float acc[4][4], acu[DUAL ? 4 : 1][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[i][j] = 0.f;
            if (DUAL) acu[i][j] = 0.f;
        }
    for (int k0 = 0; k0 < K; k0 += MK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int n = n0 + lr;
            xs[lk + i][lr] = (xrow >= 0 && k < K) ? Elem<TA>::load(x + (long)xrow * K + k) : 0.f;
            // (gate and up rows one after the other, or in alternating blocks of 32)
            const long ng = (DUAL && interleaved) ? (long)(n / 32) * 64 + n % 32 : n;
            const long nu = (DUAL && interleaved) ? ng + 32 : (long)N + n;
            ws[lk + i][lr] = (n < N && k < K) ? Elem<TW>::load(we + ng * K + k) : 0.f;
            if (DUAL) wu[lk + i][lr] = (n < N && k < K) ? Elem<TW>::load(we + nu * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MK; ++kk) {
            float a[4], b[4], c[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                b[j] = ws[kk][tx * 4 + j];
                if (DUAL) c[j] = wu[kk][tx * 4 + j];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
                    if (DUAL) acu[i][j] = fmaf(a[i], c[j], acu[i][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= rows) continue;
        if (MODE == 2) {
            TA* o = (TA*)out_ + (long)(r0 + m) * N;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n >= N) continue;
                const float z = fmaxf(acc[i][j], 0.f);
                Elem<TA>::store(o + n, z * z);
            }
        } else if (DUAL) {
            TA* o = (TA*)out_ + (long)(r0 + m) * N;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n >= N) continue;
                if (limit > 0.f) {
                    const float g = fminf(acc[i][j], limit);
                    const float u = fminf(fmaxf(acu[i][j], -limit), limit);
                    Elem<TA>::store(o + n, g / (1.f + expf(-slope * g)) * (u + 1.f));
                } else {                               // (no limit: the plain silu(g) u)
                    const float g = acc[i][j];
                    Elem<TA>::store(o + n, g / (1.f + expf(-g)) * acu[i][j]);
                }
            }
        } else {
            const int pair = perm[r0 + m];
            const float wgt = weights[pair];
            float* o = (float*)out_ + ((long)(pair % top) * T + pair / top) * N;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n < N) o[n] = wgt * acc[i][j];
            }
        }
    }
}

// dual != 0: x [T, K] rows of the pairs' tokens, w [E, 2 N, K] (gate rows then up rows, or, interleaved, in
// alternating blocks of 32), out [T * top, N] in x's type at the sorted rows.
// dual == 2: the same rows, w [E, N, K], out relu(.)^2 at the sorted rows.
// dual == 0: x [T * top, K] sorted rows, w [E, N, K], out float [top, T, N].
extern "C" int qe_moe_gemm(const void* x, const int* perm, int top, const void* w, void* out, const float* weights,
                           const int* tiles, const int* n_tiles, int max_tiles, int T, int N, int K, float limit,
                           float slope, int dual, int interleaved, int dt_a, int dt_w, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && N > 0 && K > 0 && top > 0 && max_tiles >= 0 && max_tiles <= 65535, "moe_gemm: bad sizes");
    if (T == 0 || max_tiles == 0) return 0;
    dim3 grid(qe_cdiv(N, MT), max_tiles);
#define QE_MG(TA_, TW_)                                                                                              \
    do {                                                                                                             \
        if (dual == 2) moe_gemm_kernel<TA_, TW_, 2><<<grid, 256, 0, stream>>>((const TA_*)x, perm, top, (const TW_*)w, out, weights, tiles, n_tiles, T, N, K, limit, slope, interleaved); \
        else if (dual) moe_gemm_kernel<TA_, TW_, 1><<<grid, 256, 0, stream>>>((const TA_*)x, perm, top, (const TW_*)w, out, weights, tiles, n_tiles, T, N, K, limit, slope, interleaved); \
        else moe_gemm_kernel<TA_, TW_, 0><<<grid, 256, 0, stream>>>((const TA_*)x, perm, top, (const TW_*)w, out, weights, tiles, n_tiles, T, N, K, limit, slope, interleaved);     \
    } while (0)
    if (dt_a == QE_F32 && dt_w == QE_F32) QE_MG(float, float);
    else if (dt_a == QE_BF16 && dt_w == QE_BF16) QE_MG(bf16_t, bf16_t);
    else QE_REQUIRE(false, "moe_gemm: no kernel for element types x=%d w=%d", dt_a, dt_w);
#undef QE_MG
    QE_LAUNCH_CHECK();
    return 0;
}

extern "C" int qe_moe_tile_rows() { return MT; }

template <typename TA>
__global__ void moe_gather_kernel(const TA* __restrict__ x, const int* __restrict__ perm, int top, TA* __restrict__ xs, int K) {
    const long i = blockIdx.x;
    const TA* src = x + (long)(perm[i] / top) * K;
    TA* dst = xs + i * K;
    if ((K * sizeof(TA)) % 16 == 0) {
        const int n16 = K * sizeof(TA) / 16;
        for (int c = threadIdx.x; c < n16; c += blockDim.x) ((uint4*)dst)[c] = ((const uint4*)src)[c];
    } else {
        for (int c = threadIdx.x; c < K; c += blockDim.x) dst[c] = src[c];
    }
}

extern "C" int qe_moe_gather(const void* x, const int* perm, int top, void* xs, int n, int K, int dt_a, hipStream_t stream) {
    QE_REQUIRE(n >= 0 && K > 0 && top > 0, "moe_gather: bad sizes");
    if (n == 0) return 0;
    if (dt_a == QE_BF16) moe_gather_kernel<bf16_t><<<n, 128, 0, stream>>>((const bf16_t*)x, perm, top, (bf16_t*)xs, K);
    else if (dt_a == QE_F32) moe_gather_kernel<float><<<n, 128, 0, stream>>>((const float*)x, perm, top, (float*)xs, K);
    else QE_REQUIRE(false, "moe_gather: unknown type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

template <typename TY>
__global__ void moe_combine_kernel(const TY* __restrict__ y, const int* __restrict__ inv, const float* __restrict__ weights,
                                   float* __restrict__ out, int top, int H) {
    const long t = blockIdx.x;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float a = 0.f;
        for (int j = 0; j < top; ++j) a = fmaf(weights[t * top + j], Elem<TY>::load(y + (long)inv[t * top + j] * H + c), a);
        out[t * H + c] = a;
    }
}

// y: the sorted rows, float or bfloat16 (dt_y); the sum is 32-bit either way
extern "C" int qe_moe_combine(const void* y, const int* inv, const float* weights, float* out, int T, int top, int H,
                              int dt_y, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && top > 0 && H > 0, "moe_combine: bad sizes");
    if (T == 0) return 0;
    if (dt_y == QE_F32) moe_combine_kernel<float><<<T, 256, 0, stream>>>((const float*)y, inv, weights, out, top, H);
    else if (dt_y == QE_BF16) moe_combine_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)y, inv, weights, out, top, H);
    else QE_REQUIRE(false, "moe_combine: unknown type %d", dt_y);
    QE_LAUNCH_CHECK();
    return 0;
}


// dst[t, :] (+)= sigmoid(s[t * ss]) * src[t, :]: an expert that every token uses, weighed by a gate of one number a
// token, written as one more part of the mixture's output or added to the sum that is already there.
template <typename TS>
__global__ void moe_row_gate_kernel(float* __restrict__ dst, const TS* __restrict__ src, const float* __restrict__ s, long ss,
                                    int T, int H, int accumulate) {
    const long n = (long)T * H;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const long t = i / H;
        const float g = 1.f / (1.f + expf(-s[t * ss]));
        const float v = g * Elem<TS>::load(src + i);
        dst[i] = accumulate ? dst[i] + v : v;
    }
}

extern "C" int qe_moe_row_gate(float* dst, const void* src, int dt_s, const float* s, long ss, int T, int H, int accumulate,
                               hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && ss >= 1, "moe_row_gate: bad sizes");
    if (T == 0) return 0;
    const long n = (long)T * H;
    const int blocks = (int)((n + 255) / 256 > 8192 ? 8192 : (n + 255) / 256);
    if (dt_s == QE_F32) moe_row_gate_kernel<float><<<blocks, 256, 0, stream>>>(dst, (const float*)src, s, ss, T, H, accumulate);
    else if (dt_s == QE_BF16) moe_row_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(dst, (const bf16_t*)src, s, ss, T, H, accumulate);
    else QE_REQUIRE(false, "moe_row_gate: unknown element type %d", dt_s);
    QE_LAUNCH_CHECK();
    return 0;
}
