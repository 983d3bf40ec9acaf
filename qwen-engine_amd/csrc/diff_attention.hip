// Differential attention: what stands after the attention kernels.
//
// A head has two softmax maps over the same values.  The engine runs them as two query heads against two key heads
// (the value head stored once per map), so that every attention kernel serves them: with H heads in G groups, map m
// of head h = g (H / G) + j is query head g (2 H / G) + m (H / G) + j and reads key/value head 2 g + m.  This kernel
// joins the two results:
//     o = a1 - lambda a2;   o <- o / sqrt(mean(o^2) + eps) * out_scale * sigmoid(gate[t, h])
// over a head's Dv values (the attention kernels' heads have Dc >= Dv numbers), in 32-bit, one rounding at the store.
// One wave per (token, head).
#include "common.h"

template <typename TA>
__global__ __launch_bounds__(256) void diff_heads_kernel(const TA* __restrict__ a, TA* __restrict__ out,
                                                         const TA* __restrict__ gate, long gs_t, long n_units, int H,
                                                         int G, int Dv, int Dc, float lambda, float eps, float out_scale) {
    const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n_units) return;
    const int lane = threadIdx.x & 63;
    const long t = unit / H;
    const int h = (int)(unit - t * H);
    const int per = H / G, g = h / per, j = h - g * per;
    const TA* a1 = a + (t * 2 * H + (long)g * 2 * per + j) * Dc;
    const TA* a2 = a1 + (long)per * Dc;
    float ss = 0.f;
    for (int d = lane; d < Dv; d += 64) {
        const float v = Elem<TA>::load(a1 + d) - lambda * Elem<TA>::load(a2 + d);
        ss += v * v;
    }
    ss = wave_sum(ss);
    float f = rsqrtf(ss / (float)Dv + eps) * out_scale;
    if (gate) f *= 1.f / (1.f + expf(-Elem<TA>::load(gate + t * gs_t + h)));
    TA* o = out + unit * Dv;
    for (int d = lane; d < Dv; d += 64) {
        const float v = Elem<TA>::load(a1 + d) - lambda * Elem<TA>::load(a2 + d);
        Elem<TA>::store(o + d, v * f);
    }
}

// a [T, 2 H, Dc] in the order described above; out [T, H, Dv]; gate (may be null): the number of token t and head h
// at gate[t gs_t + h].
extern "C" int qe_diff_heads(const void* a, void* out, const void* gate, long gs_t, int T, int H, int G, int Dv, int Dc,
                             float lambda, float eps, float out_scale, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0 && Dv > 0 && Dc >= Dv, "diff_heads: bad sizes H=%d G=%d Dv=%d Dc=%d",
               H, G, Dv, Dc);
    if (T == 0) return 0;
    const long n = (long)T * H;
    const int blocks = (int)((n + 3) / 4);
    if (dt_a == QE_F32)
        diff_heads_kernel<float><<<blocks, 256, 0, stream>>>((const float*)a, (float*)out, (const float*)gate, gs_t, n, H, G,
                                                              Dv, Dc, lambda, eps, out_scale);
    else if (dt_a == QE_BF16)
        diff_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)a, (bf16_t*)out, (const bf16_t*)gate, gs_t, n, H,
                                                               G, Dv, Dc, lambda, eps, out_scale);
    else
        QE_REQUIRE(false, "diff_heads: unknown element type %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}
