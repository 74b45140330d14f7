// The gated delta rule: a matrix state per head that is decayed, then corrected towards the new value.
//
//   c = silu(conv(u))                     per channel over time, J taps, the request's last J - 1 rows kept    delta_conv
//   q, k <- every head of c's q and k parts as a unit vector (x / sqrt(sum x^2 + unit_eps)), q times q_scale
//   beta = sigmoid(b),  g = exp(-exp(A_log) softplus(a + dt_bias))     one of each per token and head         delta_scan
//   S <- g S;  w = beta (v - S^T k);  S <- S + k w^T;  o = S^T q       S [key, value] float32, per head
//   y = o / rms(o) * norm_w * silu(gate)  per head, eps inside the root                                       delta_out_norm
//
// Value head h reads the q and k of head h / (H / G).  Every value channel of a head is a recurrence of its
// own over a vector of `dim` numbers (the column S[:, j]): a thread owns KI key channels of one column, the
// DELTA_IG = 16 threads of a column are neighbours in a wavefront and add up their shares of S^T k and S^T q
// through the lanes' cross-bar (no LDS, no barrier inside a token).  o is taken from the state BEFORE the
// correction: S'^T q = g S^T q + w (k . q), so both sums are taken in one pass over the column and meet the
// lanes' exchange together; k . q is made when the tokens are staged.  The state lies transposed in its row,
// [head][value][key], so a wavefront reads and writes one stretch of memory.
// All of it is 32-bit in every mode; only u, gate and y have the activation type.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define DELTA_IG 16   // threads that share a column of the state
#define DELTA_TC 8    // tokens staged at a time
#define DELTA_THREADS 256
#define DELTA_VB (DELTA_THREADS / DELTA_IG)  // value channels of a workgroup

__device__ __forceinline__ float delta_silu(float x) { return x / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------------
// Convolution, silu, unit vectors.  A row of u holds q [G dim], k [G dim], v [H vdim].  grid = (tokens,
// units / 4): a wavefront per unit (a q head, a k head or a v head), a lane keeps up to four elements.
// `state` rows hold the last J - 1 rows of u of earlier steps, oldest first (float32); zeros at admission
// stand for the zeros before a request's start.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void delta_conv_kernel(const T* __restrict__ u, int cols, const float* __restrict__ taps,
                                                          int J, const float* __restrict__ state, int64_t state_stride,
                                                          const int32_t* __restrict__ token_seq,
                                                          const int32_t* __restrict__ cu_tokens,
                                                          const int32_t* __restrict__ seq_slots, float* __restrict__ q,
                                                          float* __restrict__ k, float* __restrict__ v, int G, int dim, int H,
                                                          int vdim, float unit_eps, float q_scale) {
    const int64_t n = blockIdx.x;
    const int unit = blockIdx.y * 4 + threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    if (unit >= 2 * G + H) return;
    const int seq = token_seq[n];
    const int before = (int)(n - cu_tokens[seq]);  // rows of this request in this step ahead of row n
    const float* kept = J > 1 ? state + (int64_t)seq_slots[seq] * state_stride : nullptr;
    int col0, width;
    float* dst;
    if (unit < G) {
        col0 = unit * dim, width = dim, dst = q + n * G * dim + unit * dim;
    } else if (unit < 2 * G) {
        col0 = unit * dim, width = dim, dst = k + n * G * dim + (unit - G) * dim;
    } else {
        col0 = 2 * G * dim + (unit - 2 * G) * vdim, width = vdim, dst = v + n * H * vdim + (unit - 2 * G) * vdim;
    }
    float y[4];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int e = lane + LLE_WAVE * r;
        y[r] = 0.f;
        if (e < width) {
            const int c = col0 + e;
            float acc = 0.f;
            for (int j = 0; j < J; ++j) {
                const int back = J - 1 - j;  // how many tokens back this tap reaches
                const float x = back <= before ? to_f32<T>(u[(n - back) * cols + c])
                                               : kept[(int64_t)(J - 1 - (back - before)) * cols + c];
                acc = fmaf(taps[(int64_t)c * J + j], x, acc);
            }
            y[r] = delta_silu(acc);
            ss = fmaf(y[r], y[r], ss);
        }
    }
    float f = 1.0f;
    if (unit < 2 * G) {
        ss = wave_sum(ss);
        f = 1.0f / sqrtf(ss + unit_eps);
        if (unit < G) f *= q_scale;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int e = lane + LLE_WAVE * r;
        if (e < width) dst[e] = y[r] * f;
    }
}

extern "C" int lle_delta_conv(const void* u, int cols, const void* taps, int J, const void* state, int64_t state_stride,
                              const void* token_seq, const void* cu_tokens, const void* seq_slots, void* q, void* k, void* v,
                              int N, int G, int dim, int H, int vdim, float unit_eps, float q_scale, int dtype,
                              hipStream_t stream) {
    if (N <= 0) return 0;
    if (J < 1 || (J > 1 && state == nullptr) || G <= 0 || H <= 0 || dim <= 0 || vdim <= 0 || dim > 4 * LLE_WAVE ||
        vdim > 4 * LLE_WAVE || cols != 2 * G * dim + H * vdim || (2 * G + H + 3) / 4 > 65535)
        return (int)hipErrorInvalidValue;
    const dim3 grid(N, (2 * G + H + 3) / 4);
    if (dtype == LLE_F32)
        delta_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, cols, (const float*)taps, J, (const float*)state,
                                                            state_stride, (const int32_t*)token_seq, (const int32_t*)cu_tokens,
                                                            (const int32_t*)seq_slots, (float*)q, (float*)k, (float*)v, G, dim,
                                                            H, vdim, unit_eps, q_scale);
    else
        delta_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, cols, (const float*)taps, J,
                                                             (const float*)state, state_stride, (const int32_t*)token_seq,
                                                             (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (float*)q,
                                                             (float*)k, (float*)v, G, dim, H, vdim, unit_eps, q_scale);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// The walk.
// ---------------------------------------------------------------------------------
struct DeltaArgs {
    const float* q;        // [N, G dim]
    const float* k;        // [N, G dim]
    const float* v;        // [N, H vdim]
    const float* ba;       // [N, 2 H]: beta's input of every head, then the decay's
    const float* a_log;    // [H]
    const float* dt_bias;  // [H]
    float* state;          // rows of state_stride floats: [H][vdim][dim]
    int64_t state_stride;
    const int32_t* seq_slots;
    const int32_t* cu_tokens;
    float* out;            // [N, H vdim]
    int H, G, dim, vdim;
};

template <int CTRL>
__device__ __forceinline__ float delta_lanes(float x) {  // x of the lane that the pattern names
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

// the sum over the 16 lanes of a row, in every one of them (each step adds the same two numbers in both lanes)
__device__ __forceinline__ float delta_row_sum(float x) {
    x += delta_lanes<0xB1>(x);   // neighbours: lanes 1 0 3 2 of every four
    x += delta_lanes<0x4E>(x);   // lanes 2 3 0 1 of every four
    x += delta_lanes<0x141>(x);  // every eight mirrored
    x += delta_lanes<0x140>(x);  // the sixteen mirrored
    return x;
}

// grid = (requests, heads, blocks of DELTA_VB value channels).  Thread (jl, ig) = (tid / 16, tid % 16) owns the
// key channels [ig KI, (ig + 1) KI) of column j = block DELTA_VB + jl.
template <int KI>
__global__ __launch_bounds__(DELTA_THREADS) void delta_scan_kernel(DeltaArgs a) {
    constexpr int KD = KI * DELTA_IG;
    __shared__ __attribute__((aligned(16))) float s_q[DELTA_TC][KD];
    __shared__ __attribute__((aligned(16))) float s_k[DELTA_TC][KD];
    __shared__ float s_g[DELTA_TC], s_beta[DELTA_TC], s_kq[DELTA_TC];
    __shared__ float s_o[DELTA_TC][DELTA_VB];
    const int s = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, jl = tid / DELTA_IG, ig = tid % DELTA_IG;
    const int j0 = blockIdx.z * DELTA_VB, j = j0 + jl;
    const int dim = a.dim, vdim = a.vdim, H = a.H;
    const int hk = h / (H / a.G), GD = a.G * dim, HV = H * vdim;
    const int q0 = a.cu_tokens[s], q1 = a.cu_tokens[s + 1];
    if (q1 <= q0) return;
    float* col = a.state + (int64_t)a.seq_slots[s] * a.state_stride + ((int64_t)h * vdim + j) * dim + ig * KI;
    const bool live = j < vdim;
    float S[KI];
#pragma unroll
    for (int ii = 0; ii < KI; ++ii) S[ii] = (live && ig * KI + ii < dim) ? col[ii] : 0.f;
    const float decay_rate = expf(a.a_log[h]), dt_bias = a.dt_bias[h];

    for (int c0 = q0; c0 < q1; c0 += DELTA_TC) {
        const int nt = min(DELTA_TC, q1 - c0);
        __syncthreads();  // (the chunk before has been read)
        for (int idx = tid; idx < nt * KD; idx += DELTA_THREADS) {
            const int t = idx / KD, i = idx - t * KD;
            const int64_t at = (int64_t)(c0 + t) * GD + hk * dim + i;
            s_q[t][i] = i < dim ? a.q[at] : 0.f;
            s_k[t][i] = i < dim ? a.k[at] : 0.f;
        }
        if (tid < nt) {
            const float* ba = a.ba + (int64_t)(c0 + tid) * 2 * H;
            const float x = ba[H + h] + dt_bias;
            const float softplus = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
            s_beta[tid] = 1.0f / (1.0f + expf(-ba[h]));
            s_g[tid] = expf(-decay_rate * softplus);
        }
        float vv[DELTA_TC];
#pragma unroll
        for (int t = 0; t < DELTA_TC; ++t) vv[t] = (t < nt && live) ? a.v[(int64_t)(c0 + t) * HV + h * vdim + j] : 0.f;
        __syncthreads();
        {  // k . q of every token: a wavefront a token
            const int wave = tid / LLE_WAVE, lane = tid % LLE_WAVE;
            for (int t = wave; t < nt; t += DELTA_THREADS / LLE_WAVE) {
                float d = 0.f;
                for (int i = lane; i < KD; i += LLE_WAVE) d = fmaf(s_k[t][i], s_q[t][i], d);
                d = wave_sum(d);
                if (lane == 0) s_kq[t] = d;
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < DELTA_TC; ++t) {
            if (t < nt) {
                float kk[KI], qq[KI];
#pragma unroll
                for (int ii = 0; ii < KI; ++ii) {
                    kk[ii] = s_k[t][ig * KI + ii];
                    qq[ii] = s_q[t][ig * KI + ii];
                }
                float p = 0.f, r = 0.f;
#pragma unroll
                for (int ii = 0; ii < KI; ++ii) {
                    p = fmaf(S[ii], kk[ii], p);
                    r = fmaf(S[ii], qq[ii], r);
                }
                p = delta_row_sum(p);
                r = delta_row_sum(r);
                const float g = s_g[t];
                const float w = s_beta[t] * (vv[t] - g * p);
#pragma unroll
                for (int ii = 0; ii < KI; ++ii) S[ii] = fmaf(kk[ii], w, g * S[ii]);
                if (ig == 0) s_o[t][jl] = fmaf(w, s_kq[t], g * r);
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nt * DELTA_VB; idx += DELTA_THREADS) {
            const int t = idx / DELTA_VB, e = idx - t * DELTA_VB;
            if (j0 + e < vdim) a.out[(int64_t)(c0 + t) * HV + h * vdim + j0 + e] = s_o[t][e];
        }
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KI; ++ii)
            if (ig * KI + ii < dim) col[ii] = S[ii];
    }
}

extern "C" int lle_delta_max_dim(void) { return 16 * DELTA_IG; }

// q, k float32 [N, G dim] (unit vectors, q scaled), v float32 [N, H vdim], ba float32 [N, 2 H], a_log and dt_bias
// float32 [H]; state float32 rows of `state_stride` floats whose first H vdim dim hold the heads' states transposed;
// out float32 [N, H vdim]
extern "C" int lle_delta_scan(const void* q, const void* k, const void* v, const void* ba, const void* a_log,
                              const void* dt_bias, void* state, int64_t state_stride, const void* seq_slots,
                              const void* cu_tokens, void* out, int S, int H, int G, int dim, int vdim, hipStream_t stream) {
    if (S <= 0 || H <= 0) return 0;
    if (G <= 0 || H % G || dim <= 0 || dim > 16 * DELTA_IG || vdim <= 0 || H > 65535 || (vdim + DELTA_VB - 1) / DELTA_VB > 65535)
        return (int)hipErrorInvalidValue;
    DeltaArgs a{(const float*)q, (const float*)k, (const float*)v, (const float*)ba, (const float*)a_log, (const float*)dt_bias,
                (float*)state, state_stride, (const int32_t*)seq_slots, (const int32_t*)cu_tokens, (float*)out, H, G, dim, vdim};
    const dim3 grid(S, H, (vdim + DELTA_VB - 1) / DELTA_VB);
#define DELTA_CASE(KI)                                                      \
    if (dim <= KI * DELTA_IG) {                                             \
        delta_scan_kernel<KI><<<grid, DELTA_THREADS, 0, stream>>>(a);       \
        LLE_RETURN_LAUNCH_STATUS();                                         \
    }
    DELTA_CASE(1)
    DELTA_CASE(2)
    DELTA_CASE(4)
    DELTA_CASE(8)
    DELTA_CASE(16)
#undef DELTA_CASE
    return (int)hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------
// y[n, h, :] = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate): a wavefront per (token, head);
// grid = (tokens, heads / 4).  norm_w [vdim] is one weight for all heads.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void delta_out_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                              const void* __restrict__ norm_w, int norm_dtype, float eps,
                                                              T* __restrict__ out, int H, int vdim) {
    const int64_t n = blockIdx.x;
    const int h = blockIdx.y * 4 + threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    if (h >= H) return;
    const int64_t at = (n * H + h) * vdim;
    float ss = 0.f;
    for (int e = lane; e < vdim; e += LLE_WAVE) ss = fmaf(o[at + e], o[at + e], ss);
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
    for (int e = lane; e < vdim; e += LLE_WAVE)
        out[at + e] = from_f32<T>(o[at + e] * inv * load_as_f32(norm_w, e, norm_dtype) * delta_silu(to_f32<T>(gate[at + e])));
}

extern "C" int lle_delta_out_norm(const void* o, const void* gate, const void* norm_w, int norm_dtype, float eps, void* out,
                                  int N, int H, int vdim, int dtype, hipStream_t stream) {
    if (N <= 0 || H <= 0) return 0;
    if (vdim <= 0 || (H + 3) / 4 > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid(N, (H + 3) / 4);
    if (dtype == LLE_F32)
        delta_out_norm_kernel<float><<<grid, 256, 0, stream>>>((const float*)o, (const float*)gate, norm_w, norm_dtype, eps,
                                                                (float*)out, H, vdim);
    else
        delta_out_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)o, (const bf16_t*)gate, norm_w, norm_dtype, eps,
                                                                 (bf16_t*)out, H, vdim);
    LLE_RETURN_LAUNCH_STATUS();
}
