// Attention over one cached latent per token on the matrix units (bfloat16), for prompts' portions and
// for single new tokens alike.  See latent_attention.hip for what goes in and out: packed queries
// qp [T, H, R + Dr], cache rows [R + Dr] of which the first R are also the value, out [T, H, R].
//
// All heads read the same rows, so a wave's 16 columns are 16 heads of one token, and a block's four waves
// are head groups of one token (few rows in the step, or many heads) or consecutive tokens (many rows).
// The block walks the keys 32 at a time.  All its threads bring a tile from the cache into shared memory
// twice: row-major, K[key][d], the A operand of S^T = K Q^T (v_mfma_f32_16x16x32_bf16, contraction over d),
// and transposed, V^T[d][key], the A operand of O^T += V^T P^T (contraction over the 32 keys).  The
// transposed copy is what a row-major cache costs: a lane's operand wants eight keys of one d side by side.
// A thread loads four rows' 16 bytes and writes them back as eight 8-byte columns.  The keys of a tile are
// kept in the order in which the scores come out of the first product (lane row g holds keys 4 g .. 4 g + 3
// and 16 + 4 g .. 16 + 4 g + 3), so the weights go into the second product from the registers they are in.
//
// Tokens of a block that belong to different requests (the border between two portions, or single
// tokens of a batch when the step has many rows) are served one request after the other: the waves of the
// others wait at the barriers.
//
// The keys are cut into NS splits (a grid dimension; the same number for every token of the step, so a
// recorded step needs no knowledge of the positions): split s of a token group whose last position is p
// takes the keys [s L, (s + 1) L), L = ceil((p + 1) / NS) rounded up to 32.  With NS > 1 the splits' partial
// results (running maximum, sum, unnormalised output, 32-bit) go to a workspace and a second kernel merges
// them in the order of s.
//
// With a window of W keys a token at position p sees the positions p - W + 1 .. p: a token group's walk starts at
// the first position that its first row sees, and the splits cut what lies between that and the last row's position.
// With a sink (one number a head) the softmax's denominator has exp(sink) added, at the end of an uncut walk or
// where the splits are merged.
#include "attention_tile.h"

// bf16 per row of the transposed tile: 32 keys and 4 of padding, 18 words.  A thread writes eight rows that
// lie eight rows apart from its neighbour's; with 18 words a row those land 16 banks apart (with 20 words, 32:
// every write of the tile then met one of two banks and took thirty times as long).  A row starts at a
// multiple of 8 bytes, so a lane's operand of 16 bytes is read as two halves.
#define LAT_VT_PITCH 36
#define LAT_CHUNK 512         // keys whose places in the cache are looked up at a time

template <int RB, int DKC>
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ qp, bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const bf16_t* __restrict__ cache, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, int T, int H, int R, int Dk, int P, float scale,
    int TOK, int HGB, int NS, int window, const float* __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    const int dkc = (Dk + 31) / 32, rb = (R + 15) / 16;
    const int kpitch = dkc * 32 + 8;
    bf16_t* Ck = (bf16_t*)lds_raw;                 // [32][kpitch]
    bf16_t* VT = Ck + 32 * kpitch;                 // [rb * 16][LAT_VT_PITCH]
    __shared__ int rowoff[LAT_CHUNK];
    constexpr int ITEMS = (8 * DKC * 4 + 255) / 256;   // pieces of four rows by eight numbers that a thread brings per tile
    const int nitems = 8 * dkc * 4;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    const int split = blockIdx.y;
    const int HG = (H + 15) / 16;
    const int wt = wave / HGB, whg = wave % HGB;
    // (the step's last rows see the most keys: their blocks start first, so that no compute unit is left with a
    // long block at the end)
    const int t0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * TOK;
    const int t = t0 + wt;
    const int hg = blockIdx.z * HGB + whg;
    const bool unit_ok = wt < TOK && t < T && hg < HG;
    const int head = hg * 16 + n;
    const bool head_ok = unit_ok && head < H;

    bf16x8 q[DKC];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
        const int d = c * 32 + g * 8;
        q[c] = (head_ok && d < Dk) ? *(const bf16x8*)(qp + ((long)t * H + head) * Dk + d) : zero8;
    }
    float m = -INFINITY, l = 0.f;
    floatx4 acc[RB];
#pragma unroll
    for (int db = 0; db < RB; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};

    int seg = 0;
    while (seg < TOK && t0 + seg < T) {
        const int req = tok_seq[t0 + seg];
        int end = seg + 1;
        while (end < TOK && t0 + end < T && tok_seq[t0 + end] == req) ++end;
        const int kmax = positions[t0 + end - 1];                  // (positions rise within a request's rows)
        const int kfirst = window > 0 ? max(0, positions[t0 + seg] - window + 1) : 0;
        const int L = ((kmax - kfirst + NS) / NS + 31) & ~31;
        const int k0 = kfirst + split * L;
        const int k1 = min(k0 + L, kmax + 1);
        const bool mine = unit_ok && wt >= seg && wt < end;
        const int p = mine ? positions[t] : -1;
        const int plo = window > 0 ? p - window : -1;              // the keys above this position are seen
        const int* bt = block_table + (long)req * max_blocks;
        // The rows' places in the cache for up to LAT_CHUNK keys at a time, so that no load of a tile waits for
        // the block table; a tile's loads are issued before the tile before it is computed and go to shared
        // memory after it.
        for (int kc = k0; kc < k1; kc += LAT_CHUNK) {
            __syncthreads();
            for (int i = tid; i < LAT_CHUNK && kc + i < k1; i += 256) {
                const int key = kc + i;
                rowoff[i] = bt[key / P] * P + key % P;
            }
            __syncthreads();
            const int kend = min(kc + LAT_CHUNK, k1);
            uint4 r[ITEMS][4];
#define LAT_ISSUE(kk_)                                                                                   \
            _Pragma("unroll") for (int u = 0; u < ITEMS; ++u) {                                          \
                const int it = tid + 256 * u, kg = it & 7, d0 = (it >> 3) * 8;                           \
                _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                          \
                    const int key = (kk_) + kg * 4 + j;                                                  \
                    r[u][j] = make_uint4(0, 0, 0, 0);                                                    \
                    if (it < nitems && key < k1 && d0 < Dk)                                              \
                        r[u][j] = *(const uint4*)(cache + (long)rowoff[key - kc] * Dk + d0);             \
                }                                                                                        \
            }
            LAT_ISSUE(kc)
        for (int kk = kc; kk < kend; kk += 32) {
            __syncthreads();
#pragma unroll
            for (int u = 0; u < ITEMS; ++u) {
                // (eight neighbouring lanes take the eight groups of four keys at the same d: their transposed
                // writes fill a row of 64 bytes side by side)
                const int it = tid + 256 * u, kg = it & 7, d0 = (it >> 3) * 8;
                if (it >= nitems) continue;
#pragma unroll
                for (int j = 0; j < 4; ++j) *(uint4*)(Ck + (kg * 4 + j) * kpitch + d0) = r[u][j];
                if (d0 < rb * 16) {
                    const int i0 = (kg & 3) * 8 + (kg >= 4 ? 4 : 0);
                    const bool value = d0 < R;
                    const unsigned w[4][4] = {{r[u][0].x, r[u][0].y, r[u][0].z, r[u][0].w}, {r[u][1].x, r[u][1].y, r[u][1].z, r[u][1].w},
                                              {r[u][2].x, r[u][2].y, r[u][2].z, r[u][2].w}, {r[u][3].x, r[u][3].y, r[u][3].z, r[u][3].w}};
#pragma unroll
                    for (int e2 = 0; e2 < 4; ++e2) {               // the words hold d0 + 2 e2 (low half) and d0 + 2 e2 + 1 (high)
                        uint2 lo, hi;
                        lo.x = (w[0][e2] & 0xffffu) | (w[1][e2] << 16);
                        lo.y = (w[2][e2] & 0xffffu) | (w[3][e2] << 16);
                        hi.x = (w[0][e2] >> 16) | (w[1][e2] & 0xffff0000u);
                        hi.y = (w[2][e2] >> 16) | (w[3][e2] & 0xffff0000u);
                        if (!value) lo = hi = make_uint2(0, 0);
                        *(uint2*)(VT + (d0 + 2 * e2) * LAT_VT_PITCH + i0) = lo;
                        *(uint2*)(VT + (d0 + 2 * e2 + 1) * LAT_VT_PITCH + i0) = hi;
                    }
                }
            }
            __syncthreads();
            if (kk + 32 < kend) { LAT_ISSUE(kk + 32) }
            if (!mine) continue;
            floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DKC; ++c) {
                if (c < dkc) {
                    const bf16x8 a0 = *(const bf16x8*)(Ck + n * kpitch + c * 32 + g * 8);
                    const bf16x8 a1 = *(const bf16x8*)(Ck + (16 + n) * kpitch + c * 32 + g * 8);
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, q[c], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, q[c], s1, 0, 0, 0);
                }
            }
            float sv[8];
            float tmax = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int ka = kk + g * 4 + j, kb = ka + 16;
                sv[j] = (ka <= p && ka > plo && ka < k1) ? s0[j] * scale : -INFINITY;
                sv[4 + j] = (kb <= p && kb > plo && kb < k1) ? s1[j] * scale : -INFINITY;
                tmax = fmaxf(tmax, fmaxf(sv[j], sv[4 + j]));
            }
            tmax = max_over_lane_rows(tmax);
            const float mn = fmaxf(m, tmax);
            const float ref = (mn == -INFINITY) ? 0.f : mn;
            const float alpha = __expf(m - ref);
            bf16x8 pb;
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pj = __expf(sv[e] - ref);
                psum += pj;
                pb[e] = (__bf16)pj;
            }
            l = l * alpha + psum;
            m = mn;
#pragma unroll
            for (int db = 0; db < RB; ++db) {
                if (db < rb) {
                    union { bf16x8 v; uint2 h[2]; } au;
                    const bf16_t* ap = VT + (db * 16 + n) * LAT_VT_PITCH + g * 8;
                    au.h[0] = *(const uint2*)ap;
                    au.h[1] = *(const uint2*)(ap + 4);
                    const bf16x8 a = au.v;
                    acc[db] *= alpha;
                    acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[db], 0, 0, 0);
                }
            }
        }
        }
#undef LAT_ISSUE
        if (mine) {
            float ls = l;
            ls += __shfl_xor(ls, 16, 64);
            ls += __shfl_xor(ls, 32, 64);
            if (head_ok) {
                if (NS == 1) {
                    float inv = 1.f / ls;
                    if (sink) {
                        const float sk = sink[head], mt = fmaxf(m, sk), f = __expf(m - mt);
                        inv = f / (ls * f + __expf(sk - mt));
                    }
                    bf16_t* o = out + ((long)t * H + head) * R;
#pragma unroll
                    for (int db = 0; db < RB; ++db) {
                        const int d = db * 16 + g * 4;
                        if (d < R) {                       // (R is a multiple of 8: four numbers lie inside or outside together)
                            const float v[4] = {acc[db][0] * inv, acc[db][1] * inv, acc[db][2] * inv, acc[db][3] * inv};
                            Vec4<bf16_t>::store(o + d, v);
                        }
                    }
                } else {
                    const int RP = rb * 16;
                    float* pa = part_acc + (((long)t * H + head) * NS + split) * RP;
#pragma unroll
                    for (int db = 0; db < RB; ++db)
                        if (db < rb) *(floatx4*)(pa + db * 16 + g * 4) = acc[db];
                    if (g == 0) {
                        float* pm = part_ml + (((long)t * H + head) * NS + split) * 2;
                        pm[0] = m;
                        pm[1] = ls;
                    }
                }
            }
        }
        seg = end;
    }
}

// One block per (token, head): the splits' partial results, in the order of the splits.  Lane s of the first
// wave fetches split s's maximum and sum, so that the weights are there after one trip to memory; then every
// thread adds up its output numbers, eight splits' loads at a time.
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(const float* __restrict__ part_acc,
                                                                     const float* __restrict__ part_ml,
                                                                     bf16_t* __restrict__ out, int NS, int R, int RP,
                                                                     const float* __restrict__ sink, int H) {
    __shared__ float wgt[64];
    __shared__ float inv_l;
    const long th = blockIdx.x;
    const int tid = threadIdx.x;
    if (tid < 64) {
        const float* pm = part_ml + th * NS * 2;
        const float ms = tid < NS ? pm[2 * tid] : -INFINITY;
        const float ls = tid < NS ? pm[2 * tid + 1] : 0.f;
        float M = wave_max(ms);
        const float sk = sink ? sink[th % H] : -INFINITY;
        M = fmaxf(M, sk);
        const float w = ms == -INFINITY ? 0.f : __expf(ms - M);
        wgt[tid] = w;
        float L = sink ? __expf(sk - M) : 0.f;
        for (int s = 0; s < NS; ++s) L = fmaf(__shfl(w, s, 64), __shfl(ls, s, 64), L);      // in the order of the splits
        if (tid == 0) inv_l = 1.f / L;
    }
    __syncthreads();
    const float inv = inv_l;
    for (int d = tid; d < R; d += blockDim.x) {
        const float* pa = part_acc + th * NS * RP + d;
        float a = 0.f;
        int s = 0;
        for (; s + 8 <= NS; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = pa[(long)(s + u) * RP];
#pragma unroll
            for (int u = 0; u < 8; ++u) a = fmaf(wgt[s + u], v[u], a);
        }
        for (; s < NS; ++s) a = fmaf(wgt[s], pa[(long)s * RP], a);
        Elem<bf16_t>::store(out + th * R + d, a * inv);
    }
}

static bool latent_mfma_fits(int R, int Dk, int& rbc, int& dkc) {
    if (R <= 0 || Dk < R || R % 8 || Dk % 8) return false;
    const int rb = (R + 15) / 16, dk = (Dk + 31) / 32;
    if (rb <= 4 && dk <= 4) { rbc = 4; dkc = 4; return true; }
    if (rb <= 8 && dk <= 6) { rbc = 8; dkc = 6; return true; }
    if (rb <= 16 && dk <= 10) { rbc = 16; dkc = 10; return true; }
    if (rb <= 32 && dk <= 20) { rbc = 32; dkc = 20; return true; }
    return false;
}

extern "C" int qe_latent_attention_mfma_supported(int R, int Dr) {
    int a, b;
    return latent_mfma_fits(R, R + Dr, a, b) ? 1 : 0;
}

// How the step's rows are laid over blocks and the keys over splits: from the shapes alone.
static void latent_plan(int T, int H, int window, int& TOK, int& HGB, int& NS) {
    const int HG = (H + 15) / 16;
    HGB = HG < 4 ? HG : 4;
    TOK = T <= 64 ? 1 : (4 / HGB > 1 ? 4 / HGB : 1);
    const long blocks = (long)qe_cdiv(T, TOK) * qe_cdiv(HG, HGB);
    // Splits: enough blocks to fill the chip, but every split of every (token, head) leaves R + 2 numbers for the
    // merge to read again, so few rows get many splits and many rows few.
    NS = 1;
    if (blocks < 256) {
        NS = qe_cdiv(256, blocks);
        int cap = T <= 64 ? 256 / T : 8;
        if (cap < 8) cap = 8;
        if (cap > 32) cap = 32;
        if (NS > cap) NS = cap;
    }
    if (window > 0) {                // (a walk is no longer than the window and the block's rows: no more splits than tiles)
        const int tiles = (window + TOK + 30) / 32;
        if (NS > tiles) NS = tiles;
    }
}

extern "C" long qe_latent_attention_mfma_workspace_bytes(int T, int H, int R, int window) {
    int TOK, HGB, NS;
    latent_plan(T, H, window, TOK, HGB, NS);
    if (NS == 1) return 0;
    const long RP = (long)((R + 15) / 16) * 16;
    return (long)T * H * NS * (RP + 2) * sizeof(float);
}

extern "C" int qe_latent_attention_mfma(const void* qp, void* out, const void* cache, const int* positions,
                                        const int* tok_seq, const int* block_table, int max_blocks, int T, int H,
                                        int R, int Dr, int P, float scale, int window, const float* sink,
                                        void* workspace, long workspace_bytes, hipStream_t stream) {
    int rbc, dkcc;
    const int Dk = R + Dr;
    QE_REQUIRE(latent_mfma_fits(R, Dk, rbc, dkcc), "latent_attention (mfma): sizes R=%d Dr=%d not taken", R, Dr);
    QE_REQUIRE(H > 0 && P > 0 && window >= 0, "latent_attention (mfma): bad sizes");
    if (T == 0) return 0;
    int TOK, HGB, NS;
    latent_plan(T, H, window, TOK, HGB, NS);
    const int HG = (H + 15) / 16;
    const long RP = (long)((R + 15) / 16) * 16;
    QE_REQUIRE(workspace_bytes >= qe_latent_attention_mfma_workspace_bytes(T, H, R, window), "latent_attention (mfma): workspace too small");
    QE_REQUIRE(NS <= 64 && qe_cdiv(HG, HGB) <= 65535, "latent_attention (mfma): grid too large");
    float* part_acc = (float*)workspace;
    float* part_ml = part_acc ? part_acc + (long)T * H * NS * RP : nullptr;
    const int dkc = (Dk + 31) / 32, rb = (R + 15) / 16;
    const size_t shmem = ((size_t)32 * (dkc * 32 + 8) + (size_t)rb * 16 * LAT_VT_PITCH) * sizeof(bf16_t);
    dim3 grid(qe_cdiv(T, TOK), NS, qe_cdiv(HG, HGB));
#define QE_LA(RB_, DKC_)                                                                                              \
    do {                                                                                                              \
        static size_t attr_bytes = 48 * 1024;          /* (what a kernel may take without asking) */                 \
        if (shmem > attr_bytes) {                                                                                     \
            hipError_t e_ = hipFuncSetAttribute((const void*)latent_attention_mfma_kernel<RB_, DKC_>,                 \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);              \
            QE_REQUIRE(e_ == hipSuccess, "latent_attention (mfma): %zu bytes of shared memory: %s", shmem,             \
                       hipGetErrorString(e_));                                                                        \
            attr_bytes = shmem;                                                                                       \
        }                                                                                                             \
        latent_attention_mfma_kernel<RB_, DKC_><<<grid, 256, shmem, stream>>>(                                        \
            (const bf16_t*)qp, (bf16_t*)out, part_acc, part_ml, (const bf16_t*)cache, positions, tok_seq, block_table, \
            max_blocks, T, H, R, Dk, P, scale, TOK, HGB, NS, window, sink);                                                       \
    } while (0)
    if (rbc == 4) QE_LA(4, 4);
    else if (rbc == 8) QE_LA(8, 6);
    else if (rbc == 16) QE_LA(16, 10);
    else QE_LA(32, 20);
#undef QE_LA
    QE_LAUNCH_CHECK();
    if (NS > 1) {
        latent_attention_merge_kernel<<<T * H, R >= 256 ? 256 : (R >= 128 ? 128 : 64), 0, stream>>>(part_acc, part_ml, (bf16_t*)out, NS, R, (int)RP, sink, H);
        QE_LAUNCH_CHECK();
    }
    return 0;
}
