// A matrix product per head: out[t, h, :] = W_h x[t, h, :], W [H, N, K], for all heads in one launch.
// x and out are addressed with a row and a head stride of their own (in elements), so the product can
// read a part of each head of a wider tensor and write into a part of each head of another (the
// unrotated part of the queries into the packed queries).  With ``gate`` (the activation type; the
// number for token t, head h, output n at gate[t gs_t + h gs_h + n gs_n]: a number per output, or, with gs_n = 0,
// one per head) the result is multiplied by sigmoid(gate) before it is stored.
//
// Any sizes, every multiply-add in IEEE 32-bit, each output summed over k in ascending order whatever
// T is.  64x64 output tile per block of 256 threads, 4x4 outputs per thread, K in steps of 16 through
// shared memory; blockIdx.z is the head.
#include "common.h"

#define HT 64
#define HK 16

template <typename TA, typename TW>
__global__ __launch_bounds__(256) void gemm_heads_kernel(
    const TA* __restrict__ x, long xs_t, long xs_h, const TW* __restrict__ w, TA* __restrict__ out, long os_t,
    long os_h, const TA* __restrict__ gate, long gs_t, long gs_h, long gs_n, int T, int N, int K) {
    __shared__ float xs[HK][HT + 4];
    __shared__ float ws[HK][HT + 4];
    const int tid = threadIdx.x;
    const int h = blockIdx.z;
    const int m0 = blockIdx.y * HT, n0 = blockIdx.x * HT;
    const int lr = tid >> 2;
    const int lk = (tid & 3) * 4;
    const int ty = tid >> 4, tx = tid & 15;
    const TA* xh = x + h * xs_h;
    const TW* wh = w + (long)h * N * K;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += HK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lr, n = n0 + lr;
            xs[lk + i][lr] = (m < T && k < K) ? Elem<TA>::load(xh + (long)m * xs_t + k) : 0.f;
            ws[lk + i][lr] = (n < N && k < K) ? Elem<TW>::load(wh + (long)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < HK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    const int H = gridDim.z;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= T) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (gate) {
                const float g = Elem<TA>::load(gate + (long)m * gs_t + h * gs_h + n * gs_n);
                v = v / (1.f + expf(-g));
            }
            Elem<TA>::store(out + (long)m * os_t + h * os_h + n, v);
        }
    }
}

extern "C" int qe_gemm_heads(const void* x, long xs_t, long xs_h, const void* w, void* out, long os_t, long os_h,
                             const void* gate, long gs_t, long gs_h, long gs_n, int T, int H, int N, int K, int dt_a,
                             int dt_w, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && N > 0 && K > 0, "gemm_heads: bad sizes T=%d H=%d N=%d K=%d", T, H, N, K);
    QE_REQUIRE(H <= 65535 && qe_cdiv(T, HT) <= 65535, "gemm_heads: too many heads or rows for one launch");
    if (T == 0) return 0;
    dim3 grid(qe_cdiv(N, HT), qe_cdiv(T, HT), H);
#define QE_GH(TA_, TW_) gemm_heads_kernel<TA_, TW_><<<grid, 256, 0, stream>>>((const TA_*)x, xs_t, xs_h, (const TW_*)w, (TA_*)out, os_t, os_h, (const TA_*)gate, gs_t, gs_h, gs_n, T, N, K)
    if (dt_a == QE_F32 && dt_w == QE_F32) QE_GH(float, float);
    else if (dt_a == QE_BF16 && dt_w == QE_BF16) QE_GH(bf16_t, bf16_t);
    else if (dt_a == QE_BF16 && dt_w == QE_F32) QE_GH(bf16_t, float);
    else QE_REQUIRE(false, "gemm_heads: no kernel for element types x=%d w=%d", dt_a, dt_w);
#undef QE_GH
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- the same on the matrix units (bfloat16, K a multiple of 8) -----------------------------------------------
// out^T[n][t] = sum_k W_h[n][k] x[t][h][k] by v_mfma_f32_16x16x32_bf16: the head's weight rows are the A operand,
// the tokens' rows the B operand, both read straight from memory in 16-byte pieces.  A block's four waves take
// NT * 16 output features each for MT * 16 tokens; blockIdx.z is the head.
typedef __attribute__((ext_vector_type(8))) __bf16 gh_bf16x8;
typedef __attribute__((ext_vector_type(4))) float gh_floatx4;

template <int MT, int NT>
__global__ __launch_bounds__(256) void gemm_heads_mfma_kernel(
    const bf16_t* __restrict__ x, long xs_t, long xs_h, const bf16_t* __restrict__ w, bf16_t* __restrict__ out, long os_t,
    long os_h, const bf16_t* __restrict__ gate, long gs_t, long gs_h, long gs_n, int T, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, nn = lane & 15;
    const int h = blockIdx.z, H = gridDim.z;
    const int n_base = blockIdx.x * 64 * NT + wave * 16 * NT;      // a wave takes NT groups of 16 features
    if (n_base >= N) return;
    const int t_base = blockIdx.y * MT * 16;
    const bf16_t* wr[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n_row = n_base + j * 16 + nn < N ? n_base + j * 16 + nn : N - 1;
        wr[j] = w + ((long)h * N + n_row) * K + g * 8;
    }
    const bf16_t* xr[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int t = t_base + i * 16 + nn;
        xr[i] = x + (long)(t < T ? t : T - 1) * xs_t + h * xs_h + g * 8;
    }
    gh_floatx4 acc[NT][MT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = gh_floatx4{0.f, 0.f, 0.f, 0.f};
    const gh_bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 32) {
        const bool kin = k0 + g * 8 < K;
        gh_bf16x8 a[NT], b[MT];
#pragma unroll
        for (int j = 0; j < NT; ++j) a[j] = kin ? *(const gh_bf16x8*)(wr[j] + k0) : zero8;
#pragma unroll
        for (int i = 0; i < MT; ++i) b[i] = kin ? *(const gh_bf16x8*)(xr[i] + k0) : zero8;
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int i = 0; i < MT; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], b[i], acc[j][i], 0, 0, 0);
    }
    // lane (g, nn) holds token t_base + i * 16 + nn at the features n_base + j * 16 + g * 4 .. + 3
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int t = t_base + i * 16 + nn;
        if (t >= T) continue;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int n0 = n_base + j * 16 + g * 4;
            bf16_t* o = out + (long)t * os_t + h * os_h + n0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n0 + e >= N) break;
                float v = acc[j][i][e];
                if (gate) {
                    const float gv = Elem<bf16_t>::load(gate + (long)t * gs_t + h * gs_h + (n0 + e) * gs_n);
                    v = v / (1.f + __expf(-gv));
                }
                Elem<bf16_t>::store(o + e, v);
            }
        }
    }
}

extern "C" int qe_gemm_heads_mfma_supported(int K, long xs_t, long xs_h) { return K > 0 && K % 8 == 0 && xs_t % 8 == 0 && xs_h % 8 == 0; }

extern "C" int qe_gemm_heads_mfma(const void* x, long xs_t, long xs_h, const void* w, void* out, long os_t, long os_h,
                                  const void* gate, long gs_t, long gs_h, long gs_n, int T, int H, int N, int K,
                                  hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && N > 0 && qe_gemm_heads_mfma_supported(K, xs_t, xs_h), "gemm_heads (mfma): sizes not taken");
    QE_REQUIRE(H <= 65535, "gemm_heads (mfma): too many heads");
    if (T == 0) return 0;
    if (T <= 32) {
        dim3 grid(qe_cdiv(N, 64), qe_cdiv(T, 16), H);
        gemm_heads_mfma_kernel<1, 1><<<grid, 256, 0, stream>>>((const bf16_t*)x, xs_t, xs_h, (const bf16_t*)w, (bf16_t*)out,
                                                             os_t, os_h, (const bf16_t*)gate, gs_t, gs_h, gs_n, T, N, K);
    } else {
        QE_REQUIRE(qe_cdiv(T, 64) <= 65535, "gemm_heads (mfma): too many rows");
        // (many rows: a wave takes 32 features for 64 tokens, six loads for eight products)
        dim3 grid(qe_cdiv(N, 128), qe_cdiv(T, 64), H);
        gemm_heads_mfma_kernel<4, 2><<<grid, 256, 0, stream>>>((const bf16_t*)x, xs_t, xs_h, (const bf16_t*)w, (bf16_t*)out,
                                                             os_t, os_h, (const bf16_t*)gate, gs_t, gs_h, gs_n, T, N, K);
    }
    QE_LAUNCH_CHECK();
    return 0;
}
