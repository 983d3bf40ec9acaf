// What stands between the q | k | v product and the attention over the paged cache, for mixers whose
// queries, keys and values are normed in other ways than per head with one weight:
//   * q and k normed over the whole projection (all heads at once, a weight per coordinate) or per head
//     (one weight of the head's size for all heads), or not at all;
//   * the values taken from their own projection, or from the keys as projected, before the keys' norm;
//   * each value head divided by its root mean square (no weight);
//   * the values blended with the values that an earlier layer left for the same token,
//     v <- (1 - lambda) v + lambda v_first, or left for later layers;
//   * the first rot_dims numbers of every q and k head rotated in half-split pairs by position * inv_freq;
//   * q written with heads of Dc numbers (zeros beyond a head's own), k and v written into the cache page of
//     the token's slot, value tiles transposed ([Dc][P], what the engine's attention kernels read) or as rows
//     ([P][Dc]).
// One block per token, or, where heads are normed by themselves and the rows are few, one block per token and group of
// heads (gridDim.y groups: a group's query heads, its key heads and its value heads; a single row's time is the length
// of the walk through it, not its bytes); the row passes through shared memory in 32-bit, all arithmetic in 32-bit,
// one rounding at the stores.
#include "common.h"

enum { QKN_NONE = 0, QKN_HEAD = 1, QKN_WHOLE = 2 };

template <typename TA>
__global__ __launch_bounds__(256) void qkv_norm_store_kernel(
    const TA* __restrict__ qkv, int row_stride, const float* __restrict__ q_w, const float* __restrict__ k_w,
    int qk_mode, float qk_eps, int values_from_keys, float v_eps, int v_norm,
    const float* __restrict__ v_blend, float* __restrict__ v_first, int v_first_write,
    const int* __restrict__ positions, const float* __restrict__ inv_freq, int rot_dims,
    const int* __restrict__ slots, TA* __restrict__ q_out, TA* __restrict__ cache,
    int HqT, int HkvT, int Dk, int Dv, int Dc, int P, int v_rows) {
    extern __shared__ float sm[];
    __shared__ float red[16];
    const long t = blockIdx.x;
    // this block's heads: all of them, or one of gridDim.y equal groups
    const int Hq = HqT / (int)gridDim.y, Hkv = HkvT / (int)gridDim.y;
    const int q0 = (int)blockIdx.y * Hq, k0 = (int)blockIdx.y * Hkv;
    const int Nq = Hq * Dk, Nk = Hkv * Dk, Nv = Hkv * Dv;
    float* sq = sm;              // Nq
    float* sk = sm + Nq;         // Nk
    float* sv = sk + Nk;         // Nv
    const TA* row = qkv + t * row_stride;
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int c = tid; c < Nq; c += nt) sq[c] = Elem<TA>::load(row + q0 * Dk + c);
    for (int c = tid; c < Nk; c += nt) sk[c] = Elem<TA>::load(row + HqT * Dk + k0 * Dk + c);
    if (!values_from_keys)
        for (int c = tid; c < Nv; c += nt) sv[c] = Elem<TA>::load(row + (HqT + HkvT) * Dk + k0 * Dv + c);
    __syncthreads();
    if (values_from_keys) {      // the keys as projected (Dv == Dk)
        for (int c = tid; c < Nv; c += nt) sv[c] = sk[c];
        __syncthreads();
    }
    // ---- q and k norm ------------------------------------------------------------------------
    if (qk_mode == QKN_WHOLE) {
        float a = 0.f, b = 0.f;
        for (int c = tid; c < Nq; c += nt) a += sq[c] * sq[c];
        for (int c = tid; c < Nk; c += nt) b += sk[c] * sk[c];
        a = block_sum(a, red);
        b = block_sum(b, red);
        const float fq = rsqrtf(a / (float)Nq + qk_eps), fk = rsqrtf(b / (float)Nk + qk_eps);
        for (int c = tid; c < Nq; c += nt) sq[c] = sq[c] * fq * q_w[c];
        for (int c = tid; c < Nk; c += nt) sk[c] = sk[c] * fk * k_w[c];
        __syncthreads();
    } else if (qk_mode == QKN_HEAD) {
        const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
        for (int h = wave; h < Hq + Hkv; h += nw) {      // (q and k heads lie one after the other in sm)
            float* hp = sm + (long)h * Dk;
            const float* w = h < Hq ? q_w : k_w;
            float a = 0.f;
            for (int d = lane; d < Dk; d += 64) a += hp[d] * hp[d];
            a = wave_sum(a);
            const float f = rsqrtf(a / (float)Dk + qk_eps);
            for (int d = lane; d < Dk; d += 64) hp[d] = hp[d] * f * w[d];
        }
        __syncthreads();
    }
    // ---- values: norm per head, blend ---------------------------------------------------------
    if (v_norm) {
        const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
        for (int h = wave; h < Hkv; h += nw) {
            float* hp = sv + (long)h * Dv;
            float a = 0.f;
            for (int d = lane; d < Dv; d += 64) a += hp[d] * hp[d];
            a = wave_sum(a);
            const float f = rsqrtf(a / (float)Dv + v_eps);
            for (int d = lane; d < Dv; d += 64) hp[d] *= f;
        }
        __syncthreads();
    }
    if (v_first) {
        float* vf = v_first + t * ((long)HkvT * Dv) + k0 * Dv;
        if (v_first_write) {
            for (int c = tid; c < Nv; c += nt) vf[c] = sv[c];
        } else {
            const float lam = v_blend[0];
            for (int c = tid; c < Nv; c += nt) sv[c] = (1.f - lam) * sv[c] + lam * vf[c];
            __syncthreads();
        }
    }
    // ---- rotation of q and k ------------------------------------------------------------------
    if (rot_dims > 0) {
        const int half = rot_dims >> 1;
        const float pos = (float)positions[t];
        for (int i = tid; i < (Hq + Hkv) * half; i += nt) {
            const int h = i / half, j = i - h * half;
            float s, c;
            sincosf(pos * inv_freq[j], &s, &c);
            float* hp = sm + (long)h * Dk;
            rotate_pair(c, s, hp[j], hp[j + half]);
        }
        __syncthreads();
    }
    // ---- stores -------------------------------------------------------------------------------
    TA* qo = q_out + (t * (long)HqT + q0) * Dc;
    for (int i = tid; i < Hq * Dc; i += nt) {
        const int h = i / Dc, d = i - h * Dc;
        Elem<TA>::store(qo + i, d < Dk ? sq[h * Dk + d] : 0.f);
    }
    const int slot = slots ? slots[t] : -1;
    if (slot < 0) return;                                  // (a row that writes nowhere)
    const long page = slot / P;
    const int off = slot % P;
    TA* kp = cache + page * (2L * HkvT * P * Dc);
    TA* vp = kp + (long)HkvT * P * Dc;
    for (int i = tid; i < Hkv * Dc; i += nt) {
        const int h = i / Dc, d = i - h * Dc;
        const long hc = h + k0;                                // the head's place among all key/value heads
        Elem<TA>::store(kp + (hc * P + off) * Dc + d, d < Dk ? sk[h * Dk + d] : 0.f);
        const float v = d < Dv ? sv[h * Dv + d] : 0.f;
        if (v_rows) Elem<TA>::store(vp + (hc * P + off) * Dc + d, v);
        else Elem<TA>::store(vp + (hc * Dc + d) * P + off, v);
    }
}

// qkv [T, row_stride] holds Hq * Dk + Hkv * Dk (+ Hkv * Dv unless values_from_keys) numbers a row.
// q_w, k_w: Hq * Dk and Hkv * Dk weights (QKN_WHOLE) or Dk each (QKN_HEAD).  v_first float32 [T, Hkv * Dv]:
// written (v_first_write) with the values after their norm, or read and blended with weight v_blend[0].
// cache [pages, 2, Hkv, P * Dc].
extern "C" int qe_qkv_norm_store(const void* qkv, int row_stride, const float* q_w, const float* k_w, int qk_mode,
                                 float qk_eps, int values_from_keys, int v_norm, float v_eps, const float* v_blend,
                                 float* v_first, int v_first_write, const int* positions, const float* inv_freq,
                                 int rot_dims, const int* slots, void* q_out, void* cache, int T, int Hq, int Hkv,
                                 int Dk, int Dv, int Dc, int P, int v_rows, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && Hq > 0 && Hkv > 0 && Dk > 0 && Dv > 0 && P > 0, "qkv_norm_store: bad sizes");
    QE_REQUIRE(Dc >= Dk && Dc >= Dv, "qkv_norm_store: heads of %d and %d numbers in a cache of %d", Dk, Dv, Dc);
    QE_REQUIRE(!values_from_keys || Dv == Dk, "qkv_norm_store: values from keys of another size");
    QE_REQUIRE(qk_mode == QKN_NONE || (q_w && k_w), "qkv_norm_store: a norm without weights");
    QE_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= Dk && (rot_dims == 0 || (positions && inv_freq)),
               "qkv_norm_store: a rotation of %d numbers of heads of %d", rot_dims, Dk);
    QE_REQUIRE(!v_first || v_first_write || v_blend, "qkv_norm_store: values to blend without a weight");
    const int need = Hq * Dk + Hkv * Dk + (values_from_keys ? 0 : Hkv * Dv);
    QE_REQUIRE(row_stride >= need, "qkv_norm_store: rows of %d numbers, %d needed", row_stride, need);
    if (T == 0) return 0;
    // Few rows, heads normed by themselves (or not at all): a block per token and key/value head with its query heads
    int groups = 1;
    if (qk_mode != QKN_WHOLE && T < 512 && Hkv > 1 && Hq % Hkv == 0) groups = Hkv;
    const size_t shmem = (size_t)(Hq * Dk + Hkv * Dk + Hkv * Dv) / groups * sizeof(float);
    QE_REQUIRE(shmem <= 150 * 1024, "qkv_norm_store: a row of %zu bytes does not fit shared memory", shmem);
    const dim3 grid(T, groups);
#define QE_QNS(TA_)                                                                                                  \
    do {                                                                                                             \
        if (shmem > 48 * 1024)                                                                                       \
            (void)hipFuncSetAttribute((const void*)qkv_norm_store_kernel<TA_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem); \
        qkv_norm_store_kernel<TA_><<<grid, 256, shmem, stream>>>(                                                       \
            (const TA_*)qkv, row_stride, q_w, k_w, qk_mode, qk_eps, values_from_keys, v_eps, v_norm, v_blend, v_first, \
            v_first_write, positions, inv_freq, rot_dims, slots, (TA_*)q_out, (TA_*)cache, Hq, Hkv, Dk, Dv, Dc, P,   \
            v_rows);                                                                                                 \
    } while (0)
    if (dt_a == QE_F32) QE_QNS(float);
    else if (dt_a == QE_BF16) QE_QNS(bf16_t);
    else QE_REQUIRE(false, "qkv_norm_store: unknown element type %d", dt_a);
#undef QE_QNS
    QE_LAUNCH_CHECK();
    return 0;
}
