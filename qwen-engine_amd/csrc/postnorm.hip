// Norm after the residual sum on the 32-bit stream, with one gain for all coordinates (gain_n = 1) or one
// per coordinate (gain_n = H):
//   z = alpha * x + (delta_0 + delta_1 + ...);   x <- g * z * rsqrt(mean(z^2) + eps)
// and, if asked for, a copy of the new x in the activation type (what the next products read).
// delta holds n_delta tensors [T, H] one after the other (one branch output, or partial products
// of a matrix product, or the weighted outputs of a token's experts); they are added in ascending
// order, so a row's sum does not depend on what else is in the batch.  All arithmetic in 32-bit.
//
// And the activation of the dense feed-forward that goes with this norm:
//   act(z) = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e     per row, powers element by element
#include "common.h"

// One block per row.  The first pass writes z over x (every thread its own elements), the second
// reads it back.
template <typename TA, typename TD>
__global__ void postnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int n_delta, long delta_stride,
                                float alpha, const float* __restrict__ gain, int gain_n, float eps, TA* __restrict__ act,
                                int H) {
    __shared__ float red[16];
    const long r = blockIdx.x;
    float* xr = x + r * H;
    const TD* dr = delta ? delta + r * H : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float d = 0.f;
        if (dr) {
            d = Elem<TD>::load(dr + c);
            for (int s = 1; s < n_delta; ++s) d += Elem<TD>::load(dr + s * delta_stride + c);
        }
        const float z = fmaf(alpha, xr[c], d);
        xr[c] = z;
        ss += z * z;
    }
    ss = block_sum(ss, red);
    const float f = rsqrtf(ss / (float)H + eps) * (gain_n == 1 ? gain[0] : 1.f);
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float v = gain_n == 1 ? xr[c] * f : xr[c] * f * gain[c];
        xr[c] = v;
        if (act) Elem<TA>::store(act + r * H + c, v);
    }
}

// The same for rows of up to NV * 4 * blockDim.x numbers with H % 4 == 0: the row is read once, in 16-byte
// pieces, and kept in registers (a step of few rows is a chain of short kernels, each bound by its trips to memory).
template <typename TA, typename TD, int NV>
__global__ __launch_bounds__(256) void postnorm_regs_kernel(float* __restrict__ x, const TD* __restrict__ delta, int n_delta,
                                                            long delta_stride, float alpha, const float* __restrict__ gain,
                                                            int gain_n, float eps, TA* __restrict__ act, int H) {
    __shared__ float red[16];
    const long r = blockIdx.x;
    float* xr = x + r * H;
    const TD* dr = delta ? delta + r * H : nullptr;
    float z[NV][4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (threadIdx.x + i * blockDim.x) * 4;
        if (c < H) {
            Vec4<float>::load(xr + c, z[i]);
            float d[4] = {0.f, 0.f, 0.f, 0.f};
            if (dr) {
                Vec4<TD>::load(dr + c, d);
                for (int s = 1; s < n_delta; ++s) {
                    float e[4];
                    Vec4<TD>::load(dr + s * delta_stride + c, e);
#pragma unroll
                    for (int k = 0; k < 4; ++k) d[k] += e[k];
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                z[i][k] = fmaf(alpha, z[i][k], d[k]);
                ss += z[i][k] * z[i][k];
            }
        }
    }
    ss = block_sum(ss, red);
    const float f = rsqrtf(ss / (float)H + eps) * (gain_n == 1 ? gain[0] : 1.f);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (threadIdx.x + i * blockDim.x) * 4;
        if (c < H) {
            float gv[4] = {1.f, 1.f, 1.f, 1.f};
            if (gain_n != 1) Vec4<float>::load(gain + c, gv);
#pragma unroll
            for (int k = 0; k < 4; ++k) z[i][k] = gain_n == 1 ? z[i][k] * f : z[i][k] * f * gv[k];
            Vec4<float>::store(xr + c, z[i]);
            if (act) Vec4<TA>::store(act + r * H + c, z[i]);
        }
    }
}

// dt_d: element type of delta; dt_a: of the copy (act may be null: no copy)
extern "C" int qe_postnorm(float* x, const void* delta, int n_delta, int dt_d, float alpha, const float* gain,
                           int gain_n, float eps, void* act, int dt_a, int T, int H, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0, "postnorm: bad sizes T=%d H=%d", T, H);
    QE_REQUIRE(!delta || n_delta >= 1, "postnorm: %d delta tensors", n_delta);
    QE_REQUIRE(gain_n == 1 || gain_n == H, "postnorm: %d gains for rows of %d", gain_n, H);
    if (T == 0) return 0;
    const long stride = (long)T * H;
    const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
    const bool regs = H % 4 == 0 && H <= 8192;
    const int rthreads = regs ? (((H / 4 + 63) / 64) * 64 > 256 ? 256 : ((H / 4 + 63) / 64) * 64) : 0;
    const int nv = regs ? (H / 4 + rthreads - 1) / rthreads : 0;
#define QE_PN(TA_, TD_)                                                                                                       \
    do {                                                                                                                      \
        if (regs && nv <= 2) postnorm_regs_kernel<TA_, TD_, 2><<<T, rthreads, 0, stream>>>(x, (const TD_*)delta, n_delta, stride, alpha, gain, gain_n, eps, (TA_*)act, H); \
        else if (regs) postnorm_regs_kernel<TA_, TD_, 8><<<T, rthreads, 0, stream>>>(x, (const TD_*)delta, n_delta, stride, alpha, gain, gain_n, eps, (TA_*)act, H); \
        else postnorm_kernel<TA_, TD_><<<T, threads, 0, stream>>>(x, (const TD_*)delta, n_delta, stride, alpha, gain, gain_n, eps, (TA_*)act, H); \
    } while (0)
    const int dd = delta ? dt_d : QE_F32;
    if (dt_a == QE_F32 && dd == QE_F32) QE_PN(float, float);
    else if (dt_a == QE_BF16 && dd == QE_F32) QE_PN(bf16_t, float);
    else if (dt_a == QE_BF16 && dd == QE_BF16) QE_PN(bf16_t, bf16_t);
    else QE_REQUIRE(false, "postnorm: no kernel for copy type %d with delta type %d", dt_a, dt_d);
#undef QE_PN
    QE_LAUNCH_CHECK();
    return 0;
}

// One block per row of z [T, F] (32-bit); coef = (a, b, c, e).
template <typename TA>
__global__ void polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, float eps,
                                TA* __restrict__ out, int F) {
    __shared__ float red[16];
    const long r = blockIdx.x;
    const float* zr = z + r * F;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x; c < F; c += blockDim.x) {
        const float v = zr[c], v2 = v * v, v3 = v2 * v;
        s1 += v2;
        s2 += v2 * v2;
        s3 += v3 * v3;
    }
    s1 = block_sum(s1, red);
    s2 = block_sum(s2, red);
    s3 = block_sum(s3, red);
    const float a = coef[0] * rsqrtf(s1 / (float)F + eps);
    const float b = coef[1] * rsqrtf(s2 / (float)F + eps);
    const float cc = coef[2] * rsqrtf(s3 / (float)F + eps);
    const float e = coef[3];
    for (int c = threadIdx.x; c < F; c += blockDim.x) {
        const float v = zr[c], v2 = v * v;
        Elem<TA>::store(out + r * F + c, fmaf(a, v, fmaf(b, v2, fmaf(cc, v2 * v, e))));
    }
}

extern "C" int qe_polynorm(const float* z, const float* coef, float eps, void* out, int dt_a, int T, int F,
                           hipStream_t stream) {
    QE_REQUIRE(T >= 0 && F > 0, "polynorm: bad sizes T=%d F=%d", T, F);
    if (T == 0) return 0;
    const int threads = F >= 2048 ? 512 : (F >= 512 ? 256 : 64);
    if (dt_a == QE_F32) polynorm_kernel<float><<<T, threads, 0, stream>>>(z, coef, eps, (float*)out, F);
    else if (dt_a == QE_BF16) polynorm_kernel<bf16_t><<<T, threads, 0, stream>>>(z, coef, eps, (bf16_t*)out, F);
    else QE_REQUIRE(false, "polynorm: unknown output type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}
