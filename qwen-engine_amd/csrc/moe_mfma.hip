// The experts' two matrix products over rows grouped by expert (see moe.hip) on the matrix units, bfloat16.
//
// out^T[n][m] = sum_k W_e[n][k] X[m][k] by v_mfma_f32_16x16x32_bf16 with the weights as the A operand (a lane
// loads 16 bytes of one weight row) and the rows as the B operand (16 bytes of one row of x), both straight
// from memory: a weight is read once per tile of rows, and the rows of a tile, which every wave and every
// block of the tile's expert reads again, come from the caches.  A block's four waves take 16 output
// features each (with the gate and the up rows of the same features in the first product, so that the
// activation is formed in registers); a tile has MT * 16 rows: 16 where the step has few rows (single new
// tokens: an expert then serves a row or two and the kernel is bound by reading its weights), 64 otherwise.
// K is a multiple of 8; other sizes are arbitrary.
#include "attention_tile.h"

// KSPLIT (with MT == 1, few rows): the block's four waves take the same 16 features and a quarter of K each
// (steps of 32 in turn), and wave 0 adds the four parts in the order of the waves: four times the blocks, for
// a product that is bound by streaming the weights of the few experts that a handful of tokens choose.
template <int MT, int MODE, bool KSPLIT = false>     // MODE 0: second product, weighted; 1: gate and up; 2: one matrix, squared relu
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(
    const bf16_t* __restrict__ x, const int* __restrict__ perm, int top, const bf16_t* __restrict__ w,
    void* __restrict__ out_, const float* __restrict__ weights, const int* __restrict__ tiles,
    const int* __restrict__ n_tiles, int T, int N, int K, float limit, float slope, int interleaved) {
    constexpr bool DUAL = MODE == 1, FIRST = MODE != 0;
    if ((int)blockIdx.y >= n_tiles[0]) return;
    const int e = tiles[3 * blockIdx.y], r0 = tiles[3 * blockIdx.y + 1], rows = tiles[3 * blockIdx.y + 2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, nn = lane & 15;
    const int n_base = KSPLIT ? blockIdx.x * 16 : blockIdx.x * 64 + wave * 16;
    if (n_base >= N) return;
    const int n_row = n_base + nn < N ? n_base + nn : N - 1;
    // (gate and up rows one after the other, or in alternating blocks of 32)
    const long row_g = (DUAL && interleaved) ? (long)(n_row / 32) * 64 + n_row % 32 : n_row;
    const bf16_t* wg = w + ((long)e * (DUAL ? 2 : 1) * N + row_g) * K + g * 8;
    const bf16_t* wu = wg + ((DUAL && interleaved) ? 32L : (long)N) * K;
    const bf16_t* xr[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = i * 16 + nn;
        const int mr = m < rows ? m : 0;
        const long src = FIRST ? perm[r0 + mr] / top : r0 + mr;
        xr[i] = x + src * K + g * 8;
    }
    floatx4 ag[MT], au[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) ag[i] = au[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 2
    for (int k0 = KSPLIT ? wave * 32 : 0; k0 < K; k0 += KSPLIT ? 128 : 32) {
        const bool kin = k0 + g * 8 < K;
        const bf16x8 a = kin ? *(const bf16x8*)(wg + k0) : zero8;
        bf16x8 b = zero8;
        if (DUAL && kin) b = *(const bf16x8*)(wu + k0);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const bf16x8 xb = kin ? *(const bf16x8*)(xr[i] + k0) : zero8;
            ag[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xb, ag[i], 0, 0, 0);
            if (DUAL) au[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, xb, au[i], 0, 0, 0);
        }
    }
    if (KSPLIT) {
        __shared__ floatx4 part[3][2][64];
        if (wave > 0) {
            part[wave - 1][0][lane] = ag[0];
            if (DUAL) part[wave - 1][1][lane] = au[0];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int v = 0; v < 3; ++v) {
            ag[0] += part[v][0][lane];
            if (DUAL) au[0] += part[v][1][lane];
        }
    }
    // lane (g, nn) holds the row m = i * 16 + nn at the features n_base + g * 4 + j
    const int n0 = n_base + g * 4;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = i * 16 + nn;
        if (m >= rows) continue;
        if (MODE == 2) {
            bf16_t* o = (bf16_t*)out_ + (long)(r0 + m) * N + n0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (n0 + j >= N) break;
                const float z = fmaxf(ag[i][j], 0.f);
                Elem<bf16_t>::store(o + j, z * z);
            }
        } else if (DUAL) {
            bf16_t* o = (bf16_t*)out_ + (long)(r0 + m) * N + n0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (n0 + j >= N) break;
                if (limit > 0.f) {
                    const float gv = fminf(ag[i][j], limit);
                    const float uv = fminf(fmaxf(au[i][j], -limit), limit);
                    Elem<bf16_t>::store(o + j, gv / (1.f + __expf(-slope * gv)) * (uv + 1.f));
                } else {                               // (no limit: the plain silu(g) u)
                    const float gv = ag[i][j];
                    Elem<bf16_t>::store(o + j, gv / (1.f + __expf(-gv)) * au[i][j]);
                }
            }
        } else {
            const int pair = perm[r0 + m];
            const float wgt = weights[pair];
            float* o = (float*)out_ + ((long)(pair % top) * T + pair / top) * N + n0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n0 + j < N) o[j] = wgt * ag[i][j];
        }
    }
}

extern "C" int qe_moe_gemm_mfma_supported(int K) { return K > 0 && K % 8 == 0; }

// As qe_moe_gemm (moe.hip), bfloat16 only (dual == 2: one matrix and a squared relu); the tiles were cut with ``tile_rows`` rows (16 or 64).
extern "C" int qe_moe_gemm_mfma(const void* x, const int* perm, int top, const void* w, void* out, const float* weights,
                                const int* tiles, const int* n_tiles, int max_tiles, int tile_rows, int T, int N, int K,
                                float limit, float slope, int dual, int interleaved, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && N > 0 && top > 0 && max_tiles >= 0 && max_tiles <= 65535, "moe_gemm (mfma): bad sizes");
    QE_REQUIRE(qe_moe_gemm_mfma_supported(K), "moe_gemm (mfma): K=%d is no multiple of 8", K);
    QE_REQUIRE(tile_rows == 16 || tile_rows == 64, "moe_gemm (mfma): tiles of %d rows", tile_rows);
    if (T == 0 || max_tiles == 0) return 0;
    // few tiles of 16 rows (single new tokens): K is shared out over a block's waves
    const bool ksplit = tile_rows == 16 && max_tiles <= 64 && K >= 256;
    dim3 grid(qe_cdiv(N, ksplit ? 16 : 64), max_tiles);
#define QE_MM(MT_, DUAL_, KS_) moe_gemm_mfma_kernel<MT_, DUAL_, KS_><<<grid, 256, 0, stream>>>((const bf16_t*)x, perm, top, (const bf16_t*)w, out, weights, tiles, n_tiles, T, N, K, limit, slope, interleaved)
    if (ksplit) { if (dual == 2) QE_MM(1, 2, true); else if (dual) QE_MM(1, 1, true); else QE_MM(1, 0, true); }
    else if (tile_rows == 16) { if (dual == 2) QE_MM(1, 2, false); else if (dual) QE_MM(1, 1, false); else QE_MM(1, 0, false); }
    else { if (dual == 2) QE_MM(4, 2, false); else if (dual) QE_MM(4, 1, false); else QE_MM(4, 0, false); }
#undef QE_MM
    QE_LAUNCH_CHECK();
    return 0;
}
