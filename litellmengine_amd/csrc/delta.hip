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
#define DELTA_TC 16   // tokens staged at a time
#define DELTA_THREADS 256
#define DELTA_VB (DELTA_THREADS / DELTA_IG)  // value channels of a workgroup
static_assert(DELTA_VB == DELTA_TC, "the walk's kernel deals the staged tokens' k . q to its thread rows");

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

// The same for runs of consecutive tokens: a wavefront walks `run` tokens of one unit with the taps and the last
// J - 1 inputs of its elements in registers, so a token costs one new load per element whatever J (a workgroup a
// token re-reads J rows and the taps for every token: 61 against 25 us for 2048 tokens of 4096 channels and four
// taps).  Where the request changes inside a run the window is filled anew.
template <typename T, int J>
__global__ __launch_bounds__(256) void delta_conv_run_kernel(const T* __restrict__ u, int cols, const float* __restrict__ taps,
                                                              const float* __restrict__ state, int64_t state_stride,
                                                              const int32_t* __restrict__ token_seq,
                                                              const int32_t* __restrict__ cu_tokens,
                                                              const int32_t* __restrict__ seq_slots, float* __restrict__ q,
                                                              float* __restrict__ k, float* __restrict__ v, int N, int run, int G,
                                                              int dim, int H, int vdim, float unit_eps, float q_scale) {
    constexpr int W = J > 1 ? J - 1 : 1;
    const int unit = blockIdx.y * 4 + threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    if (unit >= 2 * G + H) return;
    const int n0 = blockIdx.x * run, n1 = min(N, n0 + run);
    int col0, width, out_cols, out0;
    float* dst;
    if (unit < G) {
        col0 = unit * dim, width = dim, dst = q, out_cols = G * dim, out0 = unit * dim;
    } else if (unit < 2 * G) {
        col0 = unit * dim, width = dim, dst = k, out_cols = G * dim, out0 = (unit - G) * dim;
    } else {
        col0 = 2 * G * dim + (unit - 2 * G) * vdim, width = vdim, dst = v, out_cols = H * vdim, out0 = (unit - 2 * G) * vdim;
    }
    float tp[4][J], win[4][W];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int e = lane + LLE_WAVE * r;
#pragma unroll
        for (int j = 0; j < J; ++j) tp[r][j] = e < width ? taps[(int64_t)(col0 + e) * J + j] : 0.f;
#pragma unroll
        for (int m = 0; m < W; ++m) win[r][m] = 0.f;
    }
    int seq_before = -1;
    for (int n = n0; n < n1; ++n) {
        const int seq = token_seq[n];
        if (J > 1 && seq != seq_before) {  // (the same for the whole wavefront) the J - 1 inputs ahead of this token
            const int before = n - cu_tokens[seq];
            const float* kept = state + (int64_t)seq_slots[seq] * state_stride;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = lane + LLE_WAVE * r;
                if (e < width) {
#pragma unroll
                    for (int m = 0; m < W; ++m) {
                        const int back = J - 1 - m;
                        win[r][m] = back <= before ? to_f32<T>(u[(int64_t)(n - back) * cols + col0 + e])
                                                   : kept[(int64_t)(J - 1 - (back - before)) * cols + col0 + e];
                    }
                }
            }
        }
        seq_before = seq;
        float y[4], ss = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int e = lane + LLE_WAVE * r;
            y[r] = 0.f;
            if (e < width) {
                const float x = to_f32<T>(u[(int64_t)n * cols + col0 + e]);
                float acc = 0.f;
                if (J > 1) {
#pragma unroll
                    for (int m = 0; m < W; ++m) acc = fmaf(tp[r][m], win[r][m], acc);
#pragma unroll
                    for (int m = 0; m + 1 < W; ++m) win[r][m] = win[r][m + 1];
                    win[r][W - 1] = x;
                }
                acc = fmaf(tp[r][J - 1], x, acc);
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
            if (e < width) dst[(int64_t)n * out_cols + out0 + e] = y[r] * f;
        }
    }
}

template <typename T>
static bool delta_conv_runs(const void* u, int cols, const void* taps, int J, const void* state, int64_t state_stride,
                            const void* token_seq, const void* cu_tokens, const void* seq_slots, void* q, void* k, void* v, int N,
                            int G, int dim, int H, int vdim, float unit_eps, float q_scale, hipStream_t stream) {
    const int blocks = (2 * G + H + 3) / 4;
    // runs long enough that taps and windows are loaded seldom, short enough that a prompt fills the chip
    int run = (int)((int64_t)N * blocks / 2048);
    run = run < 1 ? 1 : run > 16 ? 16 : run;
    const dim3 grid((N + run - 1) / run, blocks);
#define DELTA_CONV_CASE(JJ)                                                                                                   \
    case JJ:                                                                                                                  \
        delta_conv_run_kernel<T, JJ><<<grid, 256, 0, stream>>>(                                                               \
            (const T*)u, cols, (const float*)taps, (const float*)state, state_stride, (const int32_t*)token_seq,              \
            (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (float*)q, (float*)k, (float*)v, N, run, G, dim, H, vdim,   \
            unit_eps, q_scale);                                                                                               \
        return true;
    switch (J) {
        DELTA_CONV_CASE(1)
        DELTA_CONV_CASE(2)
        DELTA_CONV_CASE(3)
        DELTA_CONV_CASE(4)
        DELTA_CONV_CASE(5)
        DELTA_CONV_CASE(6)
        DELTA_CONV_CASE(7)
        DELTA_CONV_CASE(8)
    }
#undef DELTA_CONV_CASE
    return false;  // more taps: a workgroup a token
}

extern "C" int lle_delta_conv(const void* u, int cols, const void* taps, int J, const void* state, int64_t state_stride,
                              const void* token_seq, const void* cu_tokens, const void* seq_slots, void* q, void* k, void* v,
                              int N, int G, int dim, int H, int vdim, float unit_eps, float q_scale, int dtype,
                              hipStream_t stream) {
    if (N <= 0) return 0;
    if (J < 1 || (J > 1 && state == nullptr) || G <= 0 || H <= 0 || dim <= 0 || vdim <= 0 || dim > 4 * LLE_WAVE ||
        vdim > 4 * LLE_WAVE || cols != 2 * G * dim + H * vdim || (2 * G + H + 3) / 4 > 65535)
        return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32 ? delta_conv_runs<float>(u, cols, taps, J, state, state_stride, token_seq, cu_tokens, seq_slots, q, k, v, N, G,
                                                  dim, H, vdim, unit_eps, q_scale, stream)
                         : delta_conv_runs<bf16_t>(u, cols, taps, J, state, state_stride, token_seq, cu_tokens, seq_slots, q, k, v, N, G,
                                                   dim, H, vdim, unit_eps, q_scale, stream))
        LLE_RETURN_LAUNCH_STATUS();
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
    const float* gates;    // [N, 2 H]: decay and beta of every token and head, made ahead (or null: made in the walk)
};

// decay and beta of every token and head, for the walks of long portions: in the walk itself the exponentials and the
// logarithm of a chunk's sixteen tokens are one wavefront's work while the other three wait (a ninth of the walk's time)
__global__ __launch_bounds__(256) void delta_gates_kernel(const float* __restrict__ ba, const float* __restrict__ a_log,
                                                           const float* __restrict__ dt_bias, float* __restrict__ gates,
                                                           int64_t total, int H) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t n = idx / H;
    const int h = (int)(idx - n * H);
    const float x = ba[n * 2 * H + H + h] + dt_bias[h];
    const float softplus = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
    gates[n * 2 * H + h] = expf(-expf(a_log[h]) * softplus);
    gates[n * 2 * H + H + h] = 1.0f / (1.0f + expf(-ba[n * 2 * H + h]));
}

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

// What a thread reads of one staged token: its share of k and q, and the token's decay, beta and k . q.
template <int KI>
struct DeltaToken {
    float kk[KI], qq[KI];
    float g, beta, kq;
};

template <int KI>
__device__ __forceinline__ void delta_read(DeltaToken<KI>& d, const float* __restrict__ kt, const float* __restrict__ qt,
                                           const float4* __restrict__ par) {
    if (KI % 4 == 0) {
#pragma unroll
        for (int ii = 0; ii < KI; ii += 4) {
            const float4 a = *(const float4*)(kt + ii), b = *(const float4*)(qt + ii);
            d.kk[ii] = a.x, d.kk[ii + 1] = a.y, d.kk[ii + 2] = a.z, d.kk[ii + 3] = a.w;
            d.qq[ii] = b.x, d.qq[ii + 1] = b.y, d.qq[ii + 2] = b.z, d.qq[ii + 3] = b.w;
        }
    } else {
#pragma unroll
        for (int ii = 0; ii < KI; ++ii) {
            d.kk[ii] = kt[ii];
            d.qq[ii] = qt[ii];
        }
    }
    const float4 pr = *par;
    d.g = pr.x, d.beta = pr.y, d.kq = pr.z;
}

// One token of the walk for this thread's share of column j: both sums over the key channels in one pass, the
// lanes' exchange, the correction; returns the read-out.
template <int KI>
__device__ __forceinline__ float delta_token(float (&S)[KI], const DeltaToken<KI>& d, float v) {
    float p = 0.f, r = 0.f, gS[KI];
#pragma unroll
    for (int ii = 0; ii < KI; ++ii) {
        p = fmaf(S[ii], d.kk[ii], p);
        r = fmaf(S[ii], d.qq[ii], r);
        gS[ii] = d.g * S[ii];
    }
    p = delta_row_sum(p);
    r = delta_row_sum(r);
    const float w = d.beta * fmaf(-d.g, p, v);
#pragma unroll
    for (int ii = 0; ii < KI; ++ii) S[ii] = fmaf(d.kk[ii], w, gS[ii]);
    return fmaf(w, d.kq, d.g * r);
}

// grid = (requests, heads, blocks of DELTA_VB value channels).  Thread (jl, ig) = (tid / 16, tid % 16) owns the
// key channels [ig KI, (ig + 1) KI) of column j = block DELTA_VB + jl.  The tokens pass through LDS DELTA_TC at a
// time; the next chunk's q, k, v, beta and decay inputs are asked for before the current chunk is walked and wait
// in registers meanwhile, and inside a chunk every token's operands leave LDS one token ahead of their use.
// Measured at 2048 tokens of 32 heads of 64 x 64: everything asked for when it was needed 916 us; the next chunk
// ahead and whole chunks without a condition per token 591 us; operands read a token ahead, decay, beta and k . q
// in one 16-byte read 348 us; the chunk's values through LDS, one load a thread 294 us; q and k staged 16 bytes at a
// time 281 us; decays and betas made by a launch ahead of the walk 248 us.  Tried and not kept: all of a chunk's operands in registers before its first token
// and k . q made in the walk (378 us, and two workgroups no longer share a CU: 194 against 116 us for four
// requests of 512 tokens).
template <int KI>
__global__ __launch_bounds__(DELTA_THREADS) void delta_scan_kernel(DeltaArgs a) {
    constexpr int KD = KI * DELTA_IG;
    constexpr int PER = DELTA_TC * KD / DELTA_THREADS;  // elements of q (and of k) of a chunk that a thread fetches
    static_assert(DELTA_TC * KD % DELTA_THREADS == 0, "a chunk's q and k are dealt to the threads in equal shares");
    __shared__ __attribute__((aligned(16))) float s_q[DELTA_TC][KD];
    __shared__ __attribute__((aligned(16))) float s_k[DELTA_TC][KD];
    __shared__ float4 s_par[DELTA_TC];  // (decay, beta, k . q, -) of every staged token
    __shared__ float s_o[DELTA_TC][DELTA_VB];
    __shared__ float s_v[DELTA_TC][DELTA_VB];
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

    float fq[PER], fk[PER], fv = 0.f, fb = 0.f, fa = 0.f;  // the chunk that is on its way
    const bool wide = PER % 4 == 0 && dim == KD;  // whole heads of a multiple of 64 channels: 16 bytes a load and a store
    auto fetch = [&](int c0, int nt) {
        if (wide) {
#pragma unroll
            for (int r = 0; r + 3 < PER; r += 4) {
                const int e = (tid + DELTA_THREADS * (r / 4)) * 4, t = e / KD, i = e - t * KD;
                float4 x = float4{0.f, 0.f, 0.f, 0.f}, y = x;
                if (t < nt) {
                    const int64_t at = (int64_t)(c0 + t) * GD + hk * dim + i;
                    x = *(const float4*)(a.q + at);
                    y = *(const float4*)(a.k + at);
                }
                fq[r] = x.x, fq[r + 1] = x.y, fq[r + 2] = x.z, fq[r + 3] = x.w;
                fk[r] = y.x, fk[r + 1] = y.y, fk[r + 2] = y.z, fk[r + 3] = y.w;
            }
        } else {
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const int e = tid + DELTA_THREADS * r, t = e / KD, i = e - t * KD;
                const bool there = t < nt && i < dim;
                const int64_t at = (int64_t)(c0 + t) * GD + hk * dim + i;
                fq[r] = there ? a.q[at] : 0.f;
                fk[r] = there ? a.k[at] : 0.f;
            }
        }
        {  // the chunk's values of the workgroup's columns: one element a thread (one load a lane and token, sixteen
           // lanes asking for the same word, kept the memory pipeline busy for longer than the walk itself)
            const int t = tid / DELTA_VB, e = tid % DELTA_VB;
            fv = (t < nt && j0 + e < vdim) ? a.v[(int64_t)(c0 + t) * HV + h * vdim + j0 + e] : 0.f;
        }
        if (tid < nt) {  // (with gates made ahead: beta, then the decay itself)
            const float* ba = (a.gates ? a.gates : a.ba) + (int64_t)(c0 + tid) * 2 * H;
            fb = a.gates ? ba[H + h] : ba[h];
            fa = a.gates ? ba[h] : ba[H + h];
        }
    };
    fetch(q0, min(DELTA_TC, q1 - q0));

    for (int c0 = q0; c0 < q1; c0 += DELTA_TC) {
        const int nt = min(DELTA_TC, q1 - c0);
        __syncthreads();  // (the chunk before has been read, its results have left)
        if (wide) {
#pragma unroll
            for (int r = 0; r + 3 < PER; r += 4) {
                const int e = (tid + DELTA_THREADS * (r / 4)) * 4, t = e / KD, i = e - t * KD;
                *(float4*)&s_q[t][i] = float4{fq[r], fq[r + 1], fq[r + 2], fq[r + 3]};
                *(float4*)&s_k[t][i] = float4{fk[r], fk[r + 1], fk[r + 2], fk[r + 3]};
            }
        } else {
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const int e = tid + DELTA_THREADS * r, t = e / KD, i = e - t * KD;
                s_q[t][i] = fq[r];
                s_k[t][i] = fk[r];
            }
        }
        if (tid < nt) {
            float* par = (float*)&s_par[tid];
            if (a.gates) {
                par[0] = fa;
                par[1] = fb;
            } else {
                const float x = fa + dt_bias;
                const float softplus = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
                par[0] = expf(-decay_rate * softplus);
                par[1] = 1.0f / (1.0f + expf(-fb));
            }
        }
        s_v[tid / DELTA_VB][tid % DELTA_VB] = fv;
        if (c0 + DELTA_TC < q1) fetch(c0 + DELTA_TC, min(DELTA_TC, q1 - c0 - DELTA_TC));
        __syncthreads();
        float vv[DELTA_TC];
#pragma unroll
        for (int t = 0; t < DELTA_TC; ++t) vv[t] = s_v[t][jl];
        {  // k . q of every token: the sixteen lanes of thread row jl take token jl (DELTA_VB == DELTA_TC)
            float d = 0.f;
            for (int i = ig; i < KD; i += DELTA_IG) d = fmaf(s_k[jl][i], s_q[jl][i], d);
            d = delta_row_sum(d);
            if (ig == 0) ((float*)&s_par[jl])[2] = d;
        }
        __syncthreads();
        const float* kt = &s_k[0][ig * KI];
        const float* qt = &s_q[0][ig * KI];
        float oo[DELTA_TC];
        if (nt == DELTA_TC) {  // a whole chunk: nothing under a condition, every token's operands read a token ahead
            DeltaToken<KI> cur, nxt;
            delta_read<KI>(cur, kt, qt, &s_par[0]);
#pragma unroll
            for (int t = 0; t < DELTA_TC; ++t) {
                if (t + 1 < DELTA_TC) delta_read<KI>(nxt, kt + (t + 1) * KD, qt + (t + 1) * KD, &s_par[t + 1]);
                oo[t] = delta_token<KI>(S, cur, vv[t]);
                cur = nxt;
            }
        } else {
#pragma unroll
            for (int t = 0; t < DELTA_TC; ++t) {
                oo[t] = 0.f;
                if (t < nt) {
                    DeltaToken<KI> cur;
                    delta_read<KI>(cur, kt + t * KD, qt + t * KD, &s_par[t]);
                    oo[t] = delta_token<KI>(S, cur, vv[t]);
                }
            }
        }
        if (ig == 0) {
#pragma unroll
            for (int t = 0; t < DELTA_TC; ++t) s_o[t][jl] = oo[t];
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
// out float32 [N, H vdim]; `gates` (or null) scratch float32 [N, 2 H] for the decays and betas made ahead of the walk
extern "C" int lle_delta_scan(const void* q, const void* k, const void* v, const void* ba, const void* a_log,
                              const void* dt_bias, void* state, int64_t state_stride, const void* seq_slots,
                              const void* cu_tokens, void* out, int S, int H, int G, int dim, int vdim, void* gates, int N,
                              hipStream_t stream) {
    if (S <= 0 || H <= 0) return 0;
    if (G <= 0 || H % G || dim <= 0 || dim > 16 * DELTA_IG || vdim <= 0 || H > 65535 || (vdim + DELTA_VB - 1) / DELTA_VB > 65535)
        return (int)hipErrorInvalidValue;
    DeltaArgs a{(const float*)q, (const float*)k, (const float*)v, (const float*)ba, (const float*)a_log, (const float*)dt_bias,
                (float*)state, state_stride, (const int32_t*)seq_slots, (const int32_t*)cu_tokens, (float*)out, H, G, dim, vdim, (const float*)gates};
    if (gates != nullptr) {  // scratch float32 [N, 2 H], given for steps with long portions
        const int64_t total = (int64_t)N * H;
        delta_gates_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>((const float*)ba, (const float*)a_log,
                                                                            (const float*)dt_bias, (float*)gates, total, H);
    }
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
