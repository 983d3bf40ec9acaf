// Mixers that carry a matrix per head from token to token instead of keys and values:
//
//   qe_token_shift        n blends of every row with the row of the token before it in its request,
//                         y_s = x + (x' - x) * mu_s; what lies before a request's rows in this step comes from
//                         its state row (zeros for a new request), which then takes the request's last row
//   qe_linear_recurrence  per head, with a state S [D][Dv] in 32-bit:
//                           mode 0 (one decay per head):  S <- decay_h S + k_t v_t^T;   o_t = S^T q_t
//                           mode 1 (a decay per key channel, a bonus for the token itself):
//                                 o_t = (S + diag(u) k_t v_t^T)^T q_t;   S <- diag(w_t) S + k_t v_t^T
//                                 with w_t = exp(-exp(x_t + w0)) from the projected x_t
//   qe_gated_norm         y = o / rms(o) * weight * act(gate) * scale, the root mean square over each of
//                         `groups` equal pieces of a row (one: the whole row)
//
// Rows of a request are consecutive in the flat batch and tok_seq[t] names the request's state row, so a
// request's rows are found from tok_seq alone: the block of a request's first row walks on until tok_seq
// changes, every other block leaves at once.  Launch grids follow the number of rows alone.
// Everything is summed token by token in one fixed order: results do not depend on how a request was cut
// into steps or on what else is in the batch.  The recurrences' arithmetic is 32-bit throughout.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

// ---- blends with the token before ---------------------------------------------------------------------
// grid (T); mode 0: read the state, write y; mode 1: the rows that are their request's last write the state;
// mode 2: both (the caller knows that no two rows belong to one request)
template <typename TA>
__global__ void token_shift_kernel(const TA* __restrict__ x, const float* __restrict__ mu, int n,
                                   float* __restrict__ state, long state_stride, const int* __restrict__ tok_seq,
                                   TA* __restrict__ y, int T, int W, int mode) {
    const long t = blockIdx.x;
    const int seq = tok_seq[t];
    float* st = state + (long)seq * state_stride;
    if (mode == 1) {
        if (t + 1 < T && tok_seq[t + 1] == seq) return;
        for (int c = threadIdx.x; c < W; c += blockDim.x) st[c] = Elem<TA>::load(x + t * W + c);
        return;
    }
    const bool from_state = mode == 2 || t == 0 || tok_seq[t - 1] != seq;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float h = Elem<TA>::load(x + t * W + c);
        const float hp = from_state ? st[c] : Elem<TA>::load(x + (t - 1) * W + c);
        for (int s = 0; s < n; ++s)
            Elem<TA>::store(y + ((long)s * T + t) * W + c, fmaf(hp - h, mu[s * W + c], h));
        if (mode == 2) st[c] = h;
    }
}

extern "C" int qe_token_shift(const void* x, const float* mu, int n, float* state, long state_stride,
                              const int* tok_seq, void* y, int T, int W, int single_rows, int dt_a,
                              hipStream_t stream) {
    QE_REQUIRE(T >= 0 && W > 0 && n > 0 && state_stride >= W, "token_shift: bad sizes");
    if (T == 0) return 0;
    const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
#define QE_TS(TA_, mode_) token_shift_kernel<TA_><<<T, threads, 0, stream>>>((const TA_*)x, mu, n, state, state_stride, tok_seq, (TA_*)y, T, W, mode_)
    if (dt_a == QE_F32) { if (single_rows) QE_TS(float, 2); else { QE_TS(float, 0); QE_TS(float, 1); } }
    else if (dt_a == QE_BF16) { if (single_rows) QE_TS(bf16_t, 2); else { QE_TS(bf16_t, 0); QE_TS(bf16_t, 1); } }
    else QE_REQUIRE(false, "token_shift: unknown element type %d", dt_a);
#undef QE_TS
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- the recurrences -----------------------------------------------------------------------------------
// A block = one request's rows of this step x one head x up to 64 value columns.  Thread (dg, v): value column
// v, key channels dg * DPG .. dg * DPG + DPG - 1 of the state in registers (REC_DG groups share a column).  Tokens
// are taken REC_TB at a time: their q, k and decays go through shared memory once (activations and the decay's
// exponentials are applied there, once per token and channel), every thread adds its channels' share of the
// outputs token by token, and the groups' shares are added in the order of the groups at the end of the batch.
#define REC_TB 16
#define REC_DG 4

template <typename TA, int DPG, int MODE>
__global__ __launch_bounds__(REC_DG * 64) void linear_recurrence_kernel(
    const TA* __restrict__ q, const TA* __restrict__ k, const TA* __restrict__ v, long row_stride,
    const float* __restrict__ wx, long w_stride, const float* __restrict__ w0, const float* __restrict__ u,
    const float* __restrict__ decay, int act_silu, float* __restrict__ state, long state_stride,
    const int* __restrict__ tok_seq, float* __restrict__ out, int T, int H, int D, int Dv) {
    const int t0 = blockIdx.x;
    const int seq = tok_seq[t0];
    if (t0 > 0 && tok_seq[t0 - 1] == seq) return;          // not a request's first row (the whole block leaves)
    const int h = blockIdx.y;
    const int tid = threadIdx.x, vl = tid & 63, dg = tid >> 6;
    const int col = blockIdx.z * 64 + vl;
    const bool col_ok = col < Dv;
    const int d0 = dg * DPG;
    constexpr int DP = DPG * REC_DG;                        // channels with the padding
    __shared__ float sq[REC_TB][DP], sk[REC_TB][DP], sw[REC_TB][DP];
    __shared__ float part[REC_TB][REC_DG][64];

    float S[DPG], uu[DPG];
    float* Sp = state + (long)seq * state_stride + ((long)h * D) * Dv + col;
#pragma unroll
    for (int i = 0; i < DPG; ++i) {
        const int d = d0 + i;
        S[i] = (col_ok && d < D) ? Sp[(long)d * Dv] : 0.f;
        uu[i] = (MODE == 1 && d < D) ? u[h * D + d] : 0.f;
    }
    const float dec = MODE == 0 ? decay[h] : 0.f;

    int tb = t0;
    bool more = true;
    while (more) {
        // the batch's rows: tb .. tb + nb - 1, as far as they are this request's
        int nb = 0;
        while (nb < REC_TB && tb + nb < T && tok_seq[tb + nb] == seq) ++nb;
        more = nb == REC_TB && tb + nb < T && tok_seq[tb + nb] == seq;
        __syncthreads();                                     // (the batch before has been read)
        for (int i = tid; i < nb * DP; i += REC_DG * 64) {
            const int tt = i / DP, d = i - tt * DP;
            float a = 0.f, b = 0.f, c = 0.f;
            if (d < D) {
                const long r = (long)(tb + tt) * row_stride + h * D + d;
                a = Elem<TA>::load(q + r);
                b = Elem<TA>::load(k + r);
                if (act_silu) { a = silu_f(a); b = silu_f(b); }
                if (MODE == 1) c = expf(-expf(wx[(long)(tb + tt) * w_stride + h * D + d] + w0[h * D + d]));
            }
            sq[tt][d] = a; sk[tt][d] = b; sw[tt][d] = c;
        }
        float vv[REC_TB];
#pragma unroll
        for (int tt = 0; tt < REC_TB; ++tt) {
            vv[tt] = 0.f;
            if (tt < nb && col_ok) {
                vv[tt] = Elem<TA>::load(v + (long)(tb + tt) * row_stride + (long)h * Dv + col);
                if (act_silu) vv[tt] = silu_f(vv[tt]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < REC_TB; ++tt) {
            float o = 0.f;
            if (tt < nb) {
                const float vt = vv[tt];
#pragma unroll
                for (int i = 0; i < DPG; ++i) {
                    const float kv = sk[tt][d0 + i] * vt;
                    if (MODE == 0) {
                        S[i] = fmaf(dec, S[i], kv);
                        o = fmaf(sq[tt][d0 + i], S[i], o);
                    } else {
                        o = fmaf(sq[tt][d0 + i], fmaf(uu[i], kv, S[i]), o);
                        S[i] = fmaf(sw[tt][d0 + i], S[i], kv);
                    }
                }
            }
            part[tt][dg][vl] = o;
        }
        __syncthreads();
        for (int i = tid; i < nb * 64; i += REC_DG * 64) {
            const int tt = i >> 6, c = i & 63;
            if (blockIdx.z * 64 + c < Dv) {
                float o = part[tt][0][c];
#pragma unroll
                for (int g = 1; g < REC_DG; ++g) o += part[tt][g][c];
                out[((long)(tb + tt) * H + h) * Dv + blockIdx.z * 64 + c] = o;
            }
        }
        tb += nb;
    }
#pragma unroll
    for (int i = 0; i < DPG; ++i) {
        const int d = d0 + i;
        if (col_ok && d < D) Sp[(long)d * Dv] = S[i];
    }
}

// q, k: row t at + t * row_stride, H * D numbers; v likewise (v's own pointer), H * Dv numbers.  mode 1: q is what
// multiplies the state (the receptance), wx float32 [T, w_stride] the decays before their exponentials, w0 and u float32
// [H * D]; mode 0: decay float32 [H].  act_silu: q, k and v pass silu first.  state: row tok_seq[t] at
// + tok_seq[t] * state_stride, H * D * Dv floats.  out float32 [T, H, Dv].
extern "C" int qe_linear_recurrence(const void* q, const void* k, const void* v, long row_stride, const float* wx,
                                    long w_stride, const float* w0, const float* u, const float* decay, int mode,
                                    int act_silu, float* state, long state_stride, const int* tok_seq, float* out,
                                    int T, int H, int D, int Dv, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && D > 0 && Dv > 0, "linear_recurrence: bad sizes");
    QE_REQUIRE(D <= 256, "linear_recurrence: heads of %d key channels (at most 256)", D);
    QE_REQUIRE(mode == 0 ? decay != nullptr : (mode == 1 && wx && w0 && u), "linear_recurrence: mode %d lacks operands", mode);
    QE_REQUIRE(state_stride >= (long)H * D * Dv, "linear_recurrence: state rows overlap");
    if (T == 0) return 0;
    dim3 grid(T, H, (Dv + 63) / 64);
    const int dpg = D <= 32 ? 8 : (D <= 64 ? 16 : (D <= 128 ? 32 : 64));
#define QE_LR3(TA_, DPG_, MODE_) linear_recurrence_kernel<TA_, DPG_, MODE_><<<grid, REC_DG * 64, 0, stream>>>(              \
        (const TA_*)q, (const TA_*)k, (const TA_*)v, row_stride, wx, w_stride, w0, u, decay, act_silu, state, \
        state_stride, tok_seq, out, T, H, D, Dv)
#define QE_LR2(TA_, DPG_) do { if (mode == 0) QE_LR3(TA_, DPG_, 0); else QE_LR3(TA_, DPG_, 1); } while (0)
#define QE_LR(TA_) do { if (dpg == 8) QE_LR2(TA_, 8); else if (dpg == 16) QE_LR2(TA_, 16); else if (dpg == 32) QE_LR2(TA_, 32); else QE_LR2(TA_, 64); } while (0)
    if (dt_a == QE_F32) QE_LR(float);
    else if (dt_a == QE_BF16) QE_LR(bf16_t);
    else QE_REQUIRE(false, "linear_recurrence: unknown element type %d", dt_a);
#undef QE_LR
#undef QE_LR2
#undef QE_LR3
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- norm, gate --------------------------------------------------------------------------------------
// One block per row, a wave per group in turn; fewer groups than waves: all waves share every group's sums through
// shared memory.  gate_act: 0 none, 1 silu, 2 sigmoid.
template <typename TG, typename TO>
__global__ void gated_norm_kernel(const float* __restrict__ o, const float* __restrict__ weight,
                                  const TG* __restrict__ gate, long gate_stride, int gate_act, float eps, float scale,
                                  TO* __restrict__ y, long y_stride, int N, int groups) {
    const long t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int n = N / groups;
    if (groups < nw) {
        __shared__ float part[16];
        for (int g = 0; g < groups; ++g) {
            const float* og = o + t * N + (long)g * n;
            float a = 0.f;
            for (int c = threadIdx.x; c < n; c += blockDim.x) a += og[c] * og[c];
            a = wave_sum(a);
            __syncthreads();                                 // (the group before has been read)
            if (lane == 0) part[wave] = a;
            __syncthreads();
            float all = 0.f;
            for (int w = 0; w < nw; ++w) all += part[w];     // (every thread adds in the order of the waves)
            const float f = rsqrtf(all / (float)n + eps);
            for (int c = threadIdx.x; c < n; c += blockDim.x) {
                const int cc = g * n + c;
                float val = og[c] * f * weight[cc];
                if (gate) {
                    const float z = Elem<TG>::load(gate + t * gate_stride + cc);
                    val *= gate_act == 1 ? silu_f(z) : (gate_act == 2 ? sigmoid_f(z) : z);
                }
                Elem<TO>::store(y + t * y_stride + cc, val * scale);
            }
        }
        return;
    }
    for (int g = wave; g < groups; g += nw) {
        const float* og = o + t * N + (long)g * n;
        float a = 0.f;
        for (int c = lane; c < n; c += 64) a += og[c] * og[c];
        a = wave_sum(a);
        const float f = rsqrtf(a / (float)n + eps);
        for (int c = lane; c < n; c += 64) {
            const int cc = g * n + c;
            float val = og[c] * f * weight[cc];
            if (gate) {
                const float z = Elem<TG>::load(gate + t * gate_stride + cc);
                val *= gate_act == 1 ? silu_f(z) : (gate_act == 2 ? sigmoid_f(z) : z);
            }
            Elem<TO>::store(y + t * y_stride + cc, val * scale);
        }
    }
}

extern "C" int qe_gated_norm(const float* o, const float* weight, const void* gate, long gate_stride, int dt_g,
                             int gate_act, float eps, float scale, void* y, long y_stride, int dt_y, int T, int N,
                             int groups, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && N > 0 && groups > 0 && N % groups == 0, "gated_norm: rows of %d in %d groups", N, groups);
    QE_REQUIRE(y_stride >= N && (!gate || gate_stride >= N), "gated_norm: rows overlap");
    if (T == 0) return 0;
    const int threads = (groups >= 4 || N / groups >= 512) ? 256 : 64 * groups;   // (long groups: four waves share each)
#define QE_GN(TG_, TO_) gated_norm_kernel<TG_, TO_><<<T, threads, 0, stream>>>(o, weight, (const TG_*)gate, gate_stride, gate_act, eps, scale, (TO_*)y, y_stride, N, groups)
    const int dg = gate ? dt_g : dt_y;
    if (dg == QE_F32 && dt_y == QE_F32) QE_GN(float, float);
    else if (dg == QE_BF16 && dt_y == QE_BF16) QE_GN(bf16_t, bf16_t);
    else if (dg == QE_F32 && dt_y == QE_BF16) QE_GN(float, bf16_t);
    else QE_REQUIRE(false, "gated_norm: no kernel for gate type %d with output type %d", dt_g, dt_y);
#undef QE_GN
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- activations between two products, and what is done to the logits ------------------------------------
// kind 0: exact gelu, 0.5 z (1 + erf(z / sqrt 2)); 1: tanh; 2: cap * tanh(z / cap); 3: a * x + b * y
template <typename TI, typename TO>
__global__ void unary_kernel(const TI* __restrict__ z, TO* __restrict__ y, long n, int kind, float cap) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = Elem<TI>::load(z + i);
    float r;
    if (kind == 0) r = 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    else if (kind == 1) r = tanhf(v);
    else r = cap * tanhf(v / cap);
    Elem<TO>::store(y + i, r);
}

extern "C" int qe_unary(const void* z, int dt_z, void* y, int dt_y, long n, int kind, float cap, hipStream_t stream) {
    QE_REQUIRE(n >= 0 && kind >= 0 && kind <= 2, "unary: bad arguments");
    if (n == 0) return 0;
    const int blocks = qe_cdiv(n, 256);
    if (dt_z == QE_F32 && dt_y == QE_F32) unary_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)z, (float*)y, n, kind, cap);
    else if (dt_z == QE_F32 && dt_y == QE_BF16) unary_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)z, (bf16_t*)y, n, kind, cap);
    else if (dt_z == QE_BF16 && dt_y == QE_BF16) unary_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)z, (bf16_t*)y, n, kind, cap);
    else QE_REQUIRE(false, "unary: no kernel from type %d to type %d", dt_z, dt_y);
    QE_LAUNCH_CHECK();
    return 0;
}

template <typename TI>
__global__ void scaled_sum_kernel(const TI* __restrict__ a, float sa, const TI* __restrict__ b, float sb,
                                  float* __restrict__ y, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = fmaf(sb, Elem<TI>::load(b + i), sa * Elem<TI>::load(a + i));
}

extern "C" int qe_scaled_sum(const void* a, float sa, const void* b, float sb, int dt, float* y, long n,
                             hipStream_t stream) {
    QE_REQUIRE(n >= 0, "scaled_sum: bad size");
    if (n == 0) return 0;
    const int blocks = qe_cdiv(n, 256);
    if (dt == QE_F32) scaled_sum_kernel<float><<<blocks, 256, 0, stream>>>((const float*)a, sa, (const float*)b, sb, y, n);
    else if (dt == QE_BF16) scaled_sum_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)a, sa, (const bf16_t*)b, sb, y, n);
    else QE_REQUIRE(false, "scaled_sum: unknown element type %d", dt);
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- the recurrences over long portions, chunk by chunk ---------------------------------------------------
// A portion of a request's rows is cut into chunks of C rows.  With S the state before a chunk, t and s rows of the
// chunk, g_s what the chunk's remaining decays make of row s's k v^T at the chunk's end, and a_t what the decays
// before row t make of S:
//   S_out = diag(gamma) S + sum_s diag(g_s) k_s v_s^T            o_t = (q_t * a_t)^T S + sum_s A[t][s] v_s
//   one decay per head:       g_s = decay^(n-1-s), gamma = decay^n, a_t = decay^(t+1), A[t][s] = decay^(t-s) q_t . k_s (s <= t)
//   a decay per key channel:  with L_t the running sum of log w (= -exp(x + w0)) up to row t, in 64-bit:
//       g_s = exp(L_(n-1) - L_s), gamma = exp(L_(n-1)), a_t = exp(L_(t-1)),
//       A[t][s] = sum_d q_t[d] k_s[d] exp(L_(t-1)[d] - L_s[d]) (s < t),  A[t][t] = sum_d q_t[d] u[d] k_t[d]
//   (every exponent is <= 0: nothing overflows however strong the decays; log w is kept above -200, below which
//   w is 0 in 32-bit anyway, so that the running sums keep their small terms)
// Three launches: every chunk's sum_s diag(g_s) k_s v_s^T and gamma (parallel over chunks, heads and blocks of 64
// value columns); the states before every chunk, chunk after chunk within a portion (elementwise), which also leaves
// the portion's last state in the request's slot; every chunk's outputs (parallel again).
// chunks: int32 [n][2] = (first row, rows <= C); portions: int32 [m][3] = (first chunk, chunks, first row); a portion's
// state row is tok_seq of its first row, read on the device (a recorded step serves another request at every replay).
#define RC_THREADS 256

struct RecChunkLayout { int ld, d4, q, k, v, a, s, pw, l, total; };   // offsets in floats

__host__ __device__ __forceinline__ RecChunkLayout rec_chunk_layout(int C, int D, int mode) {
    RecChunkLayout L;
    L.d4 = (D + 3) & ~3;
    L.ld = L.d4 + (((L.d4 >> 2) & 1) ? 0 : 4);
    L.q = 0;
    L.k = L.q + C * L.ld;
    L.v = L.k + C * L.ld;
    L.a = L.v + C * 64;
    L.s = L.a + C * C;
    L.pw = L.s + L.d4 * 64;
    L.l = L.pw + ((C + 1 + 3) & ~3);
    L.total = L.l + (mode == 1 ? 2 * C * L.d4 : 0);
    return L;
}

extern "C" int qe_recurrence_chunk_len(int D) { return D <= 64 ? 64 : (D <= 128 ? 32 : 16); }

// PHASE 0: a chunk's contribution to the state and its whole decay; PHASE 1: its outputs from the state before it
template <typename TA, int MODE, int PHASE>
__global__ __launch_bounds__(RC_THREADS) void recurrence_chunk_kernel(
    const TA* __restrict__ q, const TA* __restrict__ k, const TA* __restrict__ v, long row_stride,
    const float* __restrict__ wx, long w_stride, const float* __restrict__ w0, const float* __restrict__ u,
    const float* __restrict__ decay, int act_silu, const int* __restrict__ chunks, float* __restrict__ ws_s,
    float* __restrict__ ws_g, float* __restrict__ out, int C, int H, int D, int Dv) {
    extern __shared__ __align__(16) float sm[];
    const RecChunkLayout L = rec_chunk_layout(C, D, MODE);
    float* qs = sm + L.q;
    float* ks = sm + L.k;
    float* vs = sm + L.v;
    float* A = sm + L.a;
    float* Ss = sm + L.s;
    float* pw = sm + L.pw;
    double* Ld = (double*)(sm + L.l);
    const int c = blockIdx.x, h = blockIdx.y, z = blockIdx.z, tid = threadIdx.x;
    const int row0 = chunks[2 * c], n = chunks[2 * c + 1];
    const int col0 = z * 64;

    for (int i = tid; i < C * L.d4; i += RC_THREADS) {
        const int t = i / L.d4, d = i - t * L.d4;
        float a = 0.f, b = 0.f;
        double lw = 0.0;
        if (t < n && d < D) {
            const long r = (long)(row0 + t) * row_stride + h * D + d;
            b = Elem<TA>::load(k + r);
            if (PHASE == 1) a = Elem<TA>::load(q + r);
            if (act_silu) { a = silu_f(a); b = silu_f(b); }
            if (MODE == 1) lw = -(double)fminf(expf(wx[(long)(row0 + t) * w_stride + h * D + d] + w0[h * D + d]), 200.f);   // (exp(-200) is 0 in 32-bit)
        }
        qs[t * L.ld + d] = a;
        ks[t * L.ld + d] = b;
        if (MODE == 1) Ld[t * L.d4 + d] = lw;
    }
    for (int i = tid; i < C * 64; i += RC_THREADS) {
        const int t = i >> 6, cc = i & 63;
        float x = 0.f;
        if (t < n && col0 + cc < Dv) {
            x = Elem<TA>::load(v + (long)(row0 + t) * row_stride + (long)h * Dv + col0 + cc);
            if (act_silu) x = silu_f(x);
        }
        vs[i] = x;
    }
    if (MODE == 0 && tid == 0) {
        float x = 1.f;
        const float dec = decay[h];
        for (int i = 0; i <= C; ++i) { pw[i] = x; x *= dec; }
    }
    __syncthreads();
    if (MODE == 1) {
        for (int d = tid; d < L.d4; d += RC_THREADS) {
            double run = 0.0;
            for (int t = 0; t < C; ++t) { run += Ld[t * L.d4 + d]; Ld[t * L.d4 + d] = run; }     // (rows from n on add nothing)
        }
        __syncthreads();
    }
    const int vq = tid & 15, rq = tid >> 4;                                  // a thread's four columns and row group

    if (PHASE == 0) {
        for (int i = tid; i < C * L.d4; i += RC_THREADS) {
            const int s = i / L.d4, d = i - s * L.d4;
            float g = 0.f;
            if (s < n) g = MODE == 0 ? pw[n - 1 - s] : expf((float)(Ld[(n - 1) * L.d4 + d] - Ld[s * L.d4 + d]));
            ks[s * L.ld + d] *= g;
        }
        if (z == 0)
            for (int d = tid; d < D; d += RC_THREADS)
                ws_g[((long)c * H + h) * D + d] = MODE == 0 ? pw[n] : expf((float)Ld[(n - 1) * L.d4 + d]);
        __syncthreads();
        float* dst = ws_s + ((long)c * H + h) * D * Dv;
        for (int d0 = rq * 4; d0 < L.d4; d0 += 64) {
            float acc[4][4] = {};
            for (int s = 0; s < n; ++s) {
                const float4 kk = *(const float4*)(ks + s * L.ld + d0);
                const float4 vv = *(const float4*)(vs + s * 64 + vq * 4);
                const float ka[4] = {kk.x, kk.y, kk.z, kk.w}, va[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ka[i], va[j], acc[i][j]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = d0 + i, cc = col0 + vq * 4 + j;
                    if (d < D && cc < Dv) dst[(long)d * Dv + cc] = acc[i][j];
                }
        }
        return;
    }

    // ---- PHASE 1
    const float* src = ws_s + ((long)c * H + h) * D * Dv;                    // (the state before this chunk by now)
    for (int i = tid; i < L.d4 * 64; i += RC_THREADS) {
        const int d = i >> 6, cc = i & 63;
        Ss[i] = (d < D && col0 + cc < Dv) ? src[(long)d * Dv + col0 + cc] : 0.f;
    }
    for (int i = tid; i < C * C; i += RC_THREADS) {
        const int t = i / C, s = i - t * C;
        float a = 0.f;
        if (t < n && s <= t) {
            const float4* qt = (const float4*)(qs + t * L.ld);
            const float4* kk = (const float4*)(ks + s * L.ld);
            if (MODE == 0) {
                float x = 0.f, y = 0.f;
                for (int d = 0; d < (L.d4 >> 2); ++d) {
                    const float4 e = qt[d], f = kk[d];
                    x = fmaf(e.x, f.x, x); y = fmaf(e.y, f.y, y); x = fmaf(e.z, f.z, x); y = fmaf(e.w, f.w, y);
                }
                a = (x + y) * pw[t - s];
            } else if (s == t) {
                for (int d = 0; d < D; ++d) a = fmaf(qs[t * L.ld + d] * u[h * D + d], ks[s * L.ld + d], a);
            } else {
                const double* lt = Ld + (t - 1) * L.d4;
                const double* ls = Ld + s * L.d4;
                for (int d = 0; d < D; ++d)
                    a = fmaf(qs[t * L.ld + d] * ks[s * L.ld + d], expf((float)(lt[d] - ls[d])), a);
            }
        }
        A[i] = a;
    }
    __syncthreads();
    for (int i = tid; i < C * L.d4; i += RC_THREADS) {
        const int t = i / L.d4, d = i - t * L.d4;
        float a;
        if (MODE == 0) a = pw[t + 1];
        else a = t == 0 ? 1.f : expf((float)Ld[(t - 1) * L.d4 + d]);
        qs[t * L.ld + d] *= a;
    }
    __syncthreads();
    for (int t0 = rq * 4; t0 < C; t0 += 64) {
        if (t0 >= n) break;
        float acc[4][4] = {};
        for (int d = 0; d < L.d4; ++d) {
            const float4 sv = *(const float4*)(Ss + d * 64 + vq * 4);
            const float sa[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float x = qs[(t0 + i) * L.ld + d];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(x, sa[j], acc[i][j]);
            }
        }
        const int s_end = t0 + 4 < n ? t0 + 4 : n;
        for (int s = 0; s < s_end; ++s) {
            const float4 vv = *(const float4*)(vs + s * 64 + vq * 4);
            const float va[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float x = A[(t0 + i) * C + s];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(x, va[j], acc[i][j]);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int t = t0 + i, cc = col0 + vq * 4 + j;
                if (t < n && cc < Dv) out[((long)(row0 + t) * H + h) * Dv + cc] = acc[i][j];
            }
    }
}

// grid (portions, H, blocks of 256 state numbers): S_in of every chunk replaces the chunk's contribution in ws_s
__global__ void recurrence_scan_kernel(const int* __restrict__ portions, const int* __restrict__ tok_seq,
                                       float* __restrict__ ws_s,
                                       const float* __restrict__ ws_g, float* __restrict__ state, long state_stride,
                                       int H, int D, int Dv) {
    const int e = blockIdx.z * blockDim.x + threadIdx.x;
    if (e >= D * Dv) return;
    const int pi = blockIdx.x, h = blockIdx.y, d = e / Dv;
    const int c0 = portions[3 * pi], nc = portions[3 * pi + 1], slot = tok_seq[portions[3 * pi + 2]];
    float* sp = state + (long)slot * state_stride + (long)h * D * Dv + e;
    float S = *sp;
    for (int c = c0; c < c0 + nc; ++c) {
        float* w = ws_s + ((long)c * H + h) * D * Dv + e;
        const float add = *w;
        *w = S;
        S = fmaf(ws_g[((long)c * H + h) * D + d], S, add);
    }
    *sp = S;
}

// As qe_linear_recurrence, for rows cut into chunks of C = qe_recurrence_chunk_len(D) rows on the host.  ws: float32,
// n_chunks * H * (D * Dv + D) numbers.  Rows that no chunk names are left alone.
extern "C" int qe_linear_recurrence_chunked(const void* q, const void* k, const void* v, long row_stride, const float* wx,
                                            long w_stride, const float* w0, const float* u, const float* decay, int mode,
                                            int act_silu, float* state, long state_stride, const int* tok_seq,
                                            const int* chunks, int n_chunks, const int* portions, int n_portions, float* ws, float* out,
                                            int H, int D, int Dv, int dt_a, hipStream_t stream) {
    QE_REQUIRE(n_chunks >= 0 && n_portions >= 0 && H > 0 && D > 0 && Dv > 0, "linear_recurrence: bad sizes");
    QE_REQUIRE(D <= 256, "linear_recurrence: heads of %d key channels (at most 256)", D);
    QE_REQUIRE(mode == 0 ? decay != nullptr : (mode == 1 && wx && w0 && u), "linear_recurrence: mode %d lacks operands", mode);
    QE_REQUIRE(state_stride >= (long)H * D * Dv, "linear_recurrence: state rows overlap");
    if (n_chunks == 0) return 0;
    QE_REQUIRE(ws && chunks && portions, "linear_recurrence: chunks without a workspace");
    const int C = qe_recurrence_chunk_len(D);
    const RecChunkLayout L = rec_chunk_layout(C, D, mode);
    const size_t shmem = (size_t)L.total * sizeof(float);
    QE_REQUIRE(shmem <= 150 * 1024, "linear_recurrence: %zu bytes of shared memory", shmem);
    float* ws_s = ws;
    float* ws_g = ws + (long)n_chunks * H * D * Dv;
    dim3 grid(n_chunks, H, (Dv + 63) / 64);
#define QE_RC(TA_, MODE_, PHASE_)                                                                                    \
    do {                                                                                                             \
        if (shmem > 48 * 1024)                                                                                       \
            (void)hipFuncSetAttribute((const void*)recurrence_chunk_kernel<TA_, MODE_, PHASE_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem); \
        recurrence_chunk_kernel<TA_, MODE_, PHASE_><<<grid, RC_THREADS, shmem, stream>>>(                            \
            (const TA_*)q, (const TA_*)k, (const TA_*)v, row_stride, wx, w_stride, w0, u, decay, act_silu, chunks,   \
            ws_s, ws_g, out, C, H, D, Dv);                                                                           \
    } while (0)
#define QE_RC2(TA_, PHASE_) do { if (mode == 0) QE_RC(TA_, 0, PHASE_); else QE_RC(TA_, 1, PHASE_); } while (0)
    QE_REQUIRE(dt_a == QE_F32 || dt_a == QE_BF16, "linear_recurrence: unknown element type %d", dt_a);
    if (dt_a == QE_F32) QE_RC2(float, 0); else QE_RC2(bf16_t, 0);
    recurrence_scan_kernel<<<dim3(n_portions, H, (D * Dv + 255) / 256), 256, 0, stream>>>(portions, tok_seq, ws_s, ws_g, state,
                                                                                         state_stride, H, D, Dv);
    if (dt_a == QE_F32) QE_RC2(float, 1); else QE_RC2(bf16_t, 1);
#undef QE_RC2
#undef QE_RC
    QE_LAUNCH_CHECK();
    return 0;
}
