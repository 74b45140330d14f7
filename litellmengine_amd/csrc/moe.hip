// Mixture of experts: the router's choice and the chosen experts' gated feed-forwards, with the
// experts indexed on the device (nothing about the choice travels to the host).
//
//   ids, gains = top-k of (logits + bias), gains = softmax over the chosen logits     moe_route
//   act[p]   = silu(Wg[e_p] x_n) * (Wu[e_p] x_n)      p = (token n, k-th choice)      moe_gate_up
//   out[n]   = sum_k gains[n, k] * Wd[e_(n,k)] act[(n, k)]        32-bit              moe_down
// An id from E on (E: the experts that have weights) names an identity expert: its result is its input,
// so such a pair adds gains[n, k] * x_n and takes no part in the products.
//
// Few tokens (decoding), or float32: every (token, choice) pair streams the rows of its expert's
// weights, a wavefront per output element.  Many bfloat16 tokens (prompt portions, large batches): the
// pairs are first put in the order of their experts (a counting sort on the device), then tiles of 128
// pairs of one expert go through the matrix cores against that expert's weights (moe_*_tile kernels),
// so that an expert's weights are read once per tile and not once per token; the per-pair results
// are added up per token, in the order of its choices, by a last kernel.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define MOE_MAX_TOP 32

// one wavefront per token: the `top` largest of logits + bias (the lower index wins a tie), then the softmax
// over those alone.  ids int32 [N, top], gains float32 [N, top].  Every round each lane looks through its own
// experts (lane, lane + 64, ...) for the best one not chosen yet, and the wavefront picks the best of the lanes.
// `bias` may be null; a row of `logits` holds `stride` >= E numbers, of which the first E are the experts'.
// mode 0: gains = softmax over the chosen alone; mode 1: gains = sigmoid of every chosen value, as it is.
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits,
                                                         const float* __restrict__ bias, int32_t* __restrict__ ids,
                                                         float* __restrict__ gains, int N, int E, int top, int stride,
                                                         int mode) {
    const int n = blockIdx.x * (blockDim.x / LLE_WAVE) + threadIdx.x / LLE_WAVE;
    const int lane = threadIdx.x % LLE_WAVE;
    if (n >= N) return;  // (the whole wavefront)
    const float* row = logits + (int64_t)n * stride;
    int chosen[MOE_MAX_TOP];   // the same in every lane
    float value[MOE_MAX_TOP];
    for (int k = 0; k < top; ++k) {
        int best = 0x7fffffff;
        float bv = -INFINITY;
        for (int e = lane; e < E; e += LLE_WAVE) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
            const float v = row[e] + (bias ? bias[e] : 0.f);
            if (!taken && (best == 0x7fffffff || v > bv)) {  // (e rises: an equal value later loses)
                best = e;
                bv = v;
            }
        }
#pragma unroll
        for (int o = LLE_WAVE / 2; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, LLE_WAVE);
            const int oe = __shfl_xor(best, o, LLE_WAVE);
            if (oe != 0x7fffffff && (best == 0x7fffffff || ov > bv || (ov == bv && oe < best))) {
                bv = ov;
                best = oe;
            }
        }
        chosen[k] = best;
        value[k] = bv;
    }
    if (lane != 0) return;
    if (mode == 1) {
        for (int k = 0; k < top; ++k) {
            ids[(int64_t)n * top + k] = chosen[k];
            gains[(int64_t)n * top + k] = 1.0f / (1.0f + expf(-value[k]));
        }
        return;
    }
    float sum = 0.f;
    const float largest = value[0];
    for (int k = 0; k < top; ++k) {
        value[k] = expf(value[k] - largest);
        sum += value[k];
    }
    for (int k = 0; k < top; ++k) {
        ids[(int64_t)n * top + k] = chosen[k];
        gains[(int64_t)n * top + k] = value[k] / sum;
    }
}

extern "C" int lle_moe_route(const void* logits, const void* bias, void* ids, void* gains, int N, int E, int top,
                             int stride, int mode, hipStream_t stream) {
    if (N <= 0) return 0;
    if (top <= 0 || top > MOE_MAX_TOP || top > E || stride < E || mode < 0 || mode > 1) return (int)hipErrorInvalidValue;
    moe_route_kernel<<<(N + 3) / 4, 256, 0, stream>>>((const float*)logits, (const float*)bias, (int32_t*)ids,
                                                           (float*)gains, N, E, top, stride, mode);
    LLE_RETURN_LAUNCH_STATUS();
}


// A router whose choice is limited to groups: one wavefront per token.  Scores s = softmax(logits) over ALL experts
// (`sigmoid`: the sigmoid of every logit on its own); choice scores c = s + correction (none: c = s); the experts
// form `groups` equal groups of neighbours, a group's score is the sum of its `group_top` largest c (1: its
// largest), and only the `keep` best groups' experts can be chosen (the lower index wins a tie, among groups and
// among experts); gains = s of the chosen / (their sum + 1e-20).
// Dynamic LDS: per wavefront E scores, E choice scores and `groups` group scores.
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ correction,
                                                                 int32_t* __restrict__ ids, float* __restrict__ gains,
                                                                 int N, int E, int top, int groups, int keep, int sigmoid,
                                                                 int group_top) {
    extern __shared__ float route_smem[];
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int n = min(blockIdx.x * (blockDim.x / LLE_WAVE) + wave, N - 1);  // (a wavefront past the end repeats the last token)
    float* s = route_smem + (int64_t)wave * (2 * E + groups);
    float* c = s + E;
    float* best = c + E;
    const float* row = logits + (int64_t)n * E;
    if (sigmoid) {
        for (int e = lane; e < E; e += LLE_WAVE) {
            const float x = 1.0f / (1.0f + expf(-row[e]));
            s[e] = x;
            c[e] = x + (correction ? correction[e] : 0.f);
        }
    } else {
        float big = -INFINITY;
        for (int e = lane; e < E; e += LLE_WAVE) big = fmaxf(big, row[e]);
        big = wave_max(big);
        float sum = 0.f;
        for (int e = lane; e < E; e += LLE_WAVE) {
            const float x = expf(row[e] - big);
            s[e] = x;
            sum += x;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += LLE_WAVE) {
            const float x = s[e] / sum;
            s[e] = x;
            c[e] = x + (correction ? correction[e] : 0.f);
        }
    }
    __syncthreads();
    const int size = E / groups;
    for (int g = lane; g < groups; g += LLE_WAVE) {
        // the group's largest choice scores, one after the other: each the best of those that come behind
        // the one before it in the order (larger first, among equals the lower index first)
        float worth = 0.f, pv = INFINITY;
        int pi = -1;
        for (int t = 0; t < min(group_top, size); ++t) {
            float bv = -INFINITY;
            int bi = -1;
            for (int i = 0; i < size; ++i) {
                const float v = c[g * size + i];
                const bool behind = v < pv || (v == pv && i > pi);
                if (behind && (bi < 0 || v > bv)) {
                    bv = v;
                    bi = i;
                }
            }
            if (bi < 0) break;
            worth = t == 0 ? bv : worth + bv;
            pv = bv;
            pi = bi;
        }
        best[g] = worth;
    }
    __syncthreads();
    if (keep < groups) {
        for (int g = lane; g < groups; g += LLE_WAVE) {
            int ahead = 0;  // groups that come before this one
            for (int o = 0; o < groups; ++o) ahead += (best[o] > best[g] || (best[o] == best[g] && o < g)) ? 1 : 0;
            if (ahead >= keep)
                for (int i = 0; i < size; ++i) c[g * size + i] = -INFINITY;
        }
        __syncthreads();
    }
    int chosen[MOE_MAX_TOP];  // the same in every lane
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        int pick = 0x7fffffff;
        float bv = -INFINITY;
        for (int e = lane; e < E; e += LLE_WAVE) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
            const float v = c[e];
            if (!taken && (pick == 0x7fffffff || v > bv)) {  // (e rises: an equal value later loses)
                pick = e;
                bv = v;
            }
        }
#pragma unroll
        for (int o = LLE_WAVE / 2; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, LLE_WAVE);
            const int oe = __shfl_xor(pick, o, LLE_WAVE);
            if (oe != 0x7fffffff && (pick == 0x7fffffff || ov > bv || (ov == bv && oe < pick))) {
                bv = ov;
                pick = oe;
            }
        }
        chosen[k] = pick;
        total += s[pick];
    }
    if (lane != 0) return;
    for (int k = 0; k < top; ++k) {
        ids[(int64_t)n * top + k] = chosen[k];
        gains[(int64_t)n * top + k] = s[chosen[k]] / (total + 1e-20f);
    }
}

extern "C" int lle_moe_route_grouped(const void* logits, const void* correction, void* ids, void* gains, int N, int E,
                                     int top, int groups, int keep, int sigmoid, int group_top, hipStream_t stream) {
    if (N <= 0) return 0;
    if (top <= 0 || top > MOE_MAX_TOP || top > E || groups <= 0 || E % groups || keep <= 0 || keep > groups ||
        top > keep * (E / groups) || group_top < 1)
        return (int)hipErrorInvalidValue;
    const size_t lds = (size_t)4 * (2 * E + groups) * sizeof(float);
    if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
    moe_route_grouped_kernel<<<(N + 3) / 4, 256, lds, stream>>>((const float*)logits, (const float*)correction,
                                                                   (int32_t*)ids, (float*)gains, N, E, top, groups, keep,
                                                                   sigmoid, group_top);
    LLE_RETURN_LAUNCH_STATUS();
}

typedef bf16_t wbf16x8 __attribute__((ext_vector_type(8)));

// sum over K of a[k] b[k] by one wavefront, every lane gets it; 16-byte loads where the rows allow them
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ a, const T* __restrict__ b, int K) {
    float acc = 0.f;
    const int lane = threadIdx.x % LLE_WAVE;
    if (sizeof(T) == 2 && K % 8 == 0) {
        for (int k = lane * 8; k < K; k += LLE_WAVE * 8) {
            const wbf16x8 av = *(const wbf16x8*)((const bf16_t*)a + k), bv = *(const wbf16x8*)((const bf16_t*)b + k);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc += (float)av[i] * (float)bv[i];
        }
    } else if (sizeof(T) == 4 && K % 4 == 0) {
        for (int k = lane * 4; k < K; k += LLE_WAVE * 4) {
            const float4 av = *(const float4*)((const float*)a + k), bv = *(const float4*)((const float*)b + k);
            acc += av.x * bv.x + av.y * bv.y + av.z * bv.z + av.w * bv.w;
        }
    } else {
        for (int k = lane; k < K; k += LLE_WAVE) acc += to_f32<T>(a[k]) * to_f32<T>(b[k]);
    }
    return wave_sum(acc);
}

// The experts' form.  MOE_GATED_SILU: act = silu(Wg x) * (Wu x), weights [E, 2 F, K] (gate rows, then up rows).
// MOE_PLAIN_RELU2: act = relu(Wu x)^2, weights [E, F, K].  `in_gains` (or null): the pair's gain multiplies the
// expert's INPUT, which is a factor on its first products' results; it is applied there, in 32-bit, before the
// activation (the gain then takes no part in the sum of the experts' results).
// MOE_GATED_CLAMP: the gated layout with g = min(Wg x, limit), u = clamp(Wu x, -limit, limit),
// act = g sigmoid(1.702 g) (u + 1).
#define MOE_GATED_SILU 0
#define MOE_PLAIN_RELU2 1
#define MOE_GATED_CLAMP 2

template <int FORM>
__device__ __forceinline__ float moe_gated_act(float g, float u, float limit) {
    if (FORM == MOE_GATED_CLAMP) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    return g / (1.0f + expf(-g)) * u;
}

__device__ __forceinline__ float moe_relu2(float z) {
    const float r = fmaxf(z, 0.f);
    return r * r;
}

// grid (pairs, ceil(F / 4)), 4 wavefronts: wavefront w makes act[p, f], f = 4 blockIdx.y + w
template <typename T, int FORM>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const int32_t* __restrict__ ids,
                                                           const T* __restrict__ gate_up,
                                                           const float* __restrict__ in_gains, T* __restrict__ act,
                                                           int top, int F, int K, int E, float limit) {
    const int p = blockIdx.x;
    const int f = blockIdx.y * 4 + threadIdx.x / LLE_WAVE;
    if (f >= F) return;
    const int e = ids[p];
    if (e >= E) return;  // an identity expert: nothing to multiply
    const T* xr = x + (int64_t)(p / top) * K;
    const float gain = in_gains ? in_gains[p] : 1.0f;
    if (FORM == MOE_PLAIN_RELU2) {
        const T* w = gate_up + (int64_t)e * F * K;
        const float z = gain * wave_dot<T>(xr, w + (int64_t)f * K, K);
        if (threadIdx.x % LLE_WAVE == 0) act[(int64_t)p * F + f] = from_f32<T>(moe_relu2(z));
        return;
    }
    const T* w = gate_up + (int64_t)e * 2 * F * K;
    const float g = gain * wave_dot<T>(xr, w + (int64_t)f * K, K);
    const float u = gain * wave_dot<T>(xr, w + (int64_t)(F + f) * K, K);
    if (threadIdx.x % LLE_WAVE == 0) act[(int64_t)p * F + f] = from_f32<T>(moe_gated_act<FORM>(g, u, limit));
}

// grid (tokens, ceil(H / 4)), 4 wavefronts: wavefront w makes out[n, o], o = 4 blockIdx.y + w
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const int32_t* __restrict__ ids,
                                                        const float* __restrict__ gains, const T* __restrict__ down,
                                                        const T* __restrict__ x, float* __restrict__ out, int top, int F,
                                                        int H, int E) {
    const int n = blockIdx.x;
    const int o = blockIdx.y * 4 + threadIdx.x / LLE_WAVE;
    if (o >= H) return;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        const int p = n * top + k;
        const int e = ids[p];
        const float gain = gains ? gains[p] : 1.0f;  // (no gains: they entered with the experts' inputs)
        if (e >= E) {  // (the same for the whole wavefront)
            total += gain * to_f32<T>(x[(int64_t)n * H + o]);
            continue;
        }
        const T* w = down + ((int64_t)e * H + o) * F;
        total += gain * wave_dot<T>(act + (int64_t)p * F, w, F);
    }
    if (threadIdx.x % LLE_WAVE == 0) out[(int64_t)n * H + o] = total;
}

template <typename T>
static void moe_experts_pairs(const void* x, const void* ids, const void* gains, const void* gate_up, const void* down,
                              void* act, void* out, int N, int top, int E, int F, int K, int H, int form,
                              int gain_on_input, float limit, hipStream_t stream) {
    const dim3 g1(N * top, (F + 3) / 4), g2(N, (H + 3) / 4);
    const float* in_gains = gain_on_input ? (const float*)gains : nullptr;
    const float* out_gains = gain_on_input ? nullptr : (const float*)gains;
    if (form == MOE_PLAIN_RELU2)
        moe_gate_up_kernel<T, MOE_PLAIN_RELU2><<<g1, 256, 0, stream>>>((const T*)x, (const int32_t*)ids,
                                                                         (const T*)gate_up, in_gains, (T*)act, top, F, K, E, limit);
    else if (form == MOE_GATED_CLAMP)
        moe_gate_up_kernel<T, MOE_GATED_CLAMP><<<g1, 256, 0, stream>>>((const T*)x, (const int32_t*)ids,
                                                                         (const T*)gate_up, in_gains, (T*)act, top, F, K, E, limit);
    else
        moe_gate_up_kernel<T, MOE_GATED_SILU><<<g1, 256, 0, stream>>>((const T*)x, (const int32_t*)ids,
                                                                        (const T*)gate_up, in_gains, (T*)act, top, F, K, E, limit);
    moe_down_kernel<T><<<g2, 256, 0, stream>>>((const T*)act, (const int32_t*)ids, out_gains, (const T*)down,
                                                (const T*)x, (float*)out, top, F, H, E);
}

// x [N, K], ids/gains [N, top], gate_up [E, 2 F, K] (form 0) or [E, F, K] (form 1), down [E, H, F], act [N top, F]
// (scratch), out float32 [N, H]; ids from E on are identity experts (then H = K); `gain_on_input`: the gains
// multiply the experts' inputs, not their results
extern "C" int lle_moe_experts(const void* x, const void* ids, const void* gains, const void* gate_up,
                               const void* down, void* act, void* out, int N, int top, int E, int F, int K, int H,
                               int dtype, int form, int gain_on_input, float limit, hipStream_t stream) {
    if (N <= 0) return 0;
    if (top <= 0 || (int64_t)N * top > 0x7fffffff || form < 0 || form > 2) return (int)hipErrorInvalidValue;
    if ((F + 3) / 4 > 65535 || (H + 3) / 4 > 65535) return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        moe_experts_pairs<float>(x, ids, gains, gate_up, down, act, out, N, top, E, F, K, H, form, gain_on_input, limit, stream);
    else
        moe_experts_pairs<bf16_t>(x, ids, gains, gate_up, down, act, out, N, top, E, F, K, H, form, gain_on_input, limit, stream);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// Many pairs: sorted by expert, then tiles on the matrix cores (bfloat16).
//   counts[e]            pairs of expert e                                   moe_count_kernel
//   first[e], tile0[e]   first sorted row / first 128-row tile of expert e   moe_plan_kernel (one workgroup)
//   order[row] = pair, place[pair] = row                                     moe_place_kernel
// The order of an expert's pairs among themselves is whatever the atomics give; no value depends on it.
// A tile workgroup finds its expert by walking tile0[] (at most 256 experts), and leaves if the step
// has fewer tiles than the grid (the grid is sized for the worst case, pairs / 128 + experts).
// Products as C^T = W X^T with v_mfma_f32_16x16x32_bf16: lane (c = lane / 16, r = lane % 16) loads 16
// bytes of row r of a 16-row tile of W (A) and of X (B) and holds outputs n = 4c .. 4c + 3 of row r.
// A wavefront keeps 128 rows x 64 outputs (gate_up: 128 rows x 32 gate + 32 up); four wavefronts of a
// workgroup sit side by side along the outputs and share the X rows, which pass through LDS once for all of
// them.  (Measured at 2048 tokens, 64 experts, top 6, 2048 x 1408: four wavefronts of 64 rows each against one
// shared block of W rows are 1.6 times slower than four side by side along the outputs.)
// ---------------------------------------------------------------------------------------------
#define MOE_TM 128
#define MOE_XS 40  // bfloat16 elements between the X rows in LDS: 32 of a step and 16 bytes to spread the banks
typedef bf16_t mbf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t mbf16x4 __attribute__((ext_vector_type(4)));
typedef float mf32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void moe_zero_kernel(int32_t* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// (E <= 256.)  A workgroup counts its 256 pairs in LDS first and then adds one number per expert to the global counts.
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ counts,
                                                         int pairs, int E) {
    __shared__ int32_t local[256];
    local[threadIdx.x] = 0;
    __syncthreads();
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p < pairs && ids[p] < E) atomicAdd(&local[ids[p]], 1);  // (identity experts have no rows)
    __syncthreads();
    if (threadIdx.x < E && local[threadIdx.x]) atomicAdd(&counts[threadIdx.x], local[threadIdx.x]);
}

// plan = [counts E | cursor E | first E | tile0 E + 1]
__global__ __launch_bounds__(256) void moe_plan_kernel(int32_t* __restrict__ plan, int E) {
    __shared__ int32_t counts[256];
    if (threadIdx.x < E) counts[threadIdx.x] = plan[threadIdx.x];
    __syncthreads();
    if (threadIdx.x != 0) return;
    int32_t* first = plan + 2 * E;
    int32_t* tile0 = plan + 3 * E;
    int row = 0, tile = 0;
    for (int e = 0; e < E; ++e) {
        first[e] = row;
        tile0[e] = tile;
        row += counts[e];
        tile += (counts[e] + MOE_TM - 1) / MOE_TM;
    }
    tile0[E] = tile;
}

// a workgroup numbers its pairs per expert in LDS, takes one range per expert from the global cursor, and places them
__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ plan,
                                                         int32_t* __restrict__ order, int32_t* __restrict__ place,
                                                         int pairs, int E) {
    __shared__ int32_t local[256];
    local[threadIdx.x] = 0;
    __syncthreads();
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    int e = 0, mine = 0;
    if (p < pairs) {
        e = ids[p];
        if (e < E) mine = atomicAdd(&local[e], 1);
    }
    __syncthreads();
    if (threadIdx.x < E && local[threadIdx.x])
        local[threadIdx.x] = plan[2 * E + threadIdx.x] + atomicAdd(&plan[E + threadIdx.x], local[threadIdx.x]);
    __syncthreads();
    if (p >= pairs) return;
    if (e >= E) {  // an identity expert: the pair has no row
        place[p] = -1;
        return;
    }
    const int row = local[e] + mine;
    order[row] = p;
    place[p] = row;
}

__device__ __forceinline__ mbf16x8 moe_zero8() {
    mbf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (bf16_t)0.0f;
    return z;
}

__device__ __forceinline__ mbf16x8 moe_load8(const bf16_t* row, int k, int K) {
    return (row && k < K) ? *(const mbf16x8*)(row + k) : moe_zero8();
}

// acc[nt][mt] += W rows . X rows over K in steps of 32, for a wavefront's 64 outputs (four 16-row tiles of W,
// straight from memory: nobody else reads them) against the workgroup's 128 X rows (eight tiles), which all four
// wavefronts share: every thread brings 32 bytes of them into LDS per step (`xrow`: its two rows, columns
// 8 (thread % 4) on; nullptr for a row that does not exist).  The operands of the next step are asked for before
// the current one is multiplied; the LDS buffers take turns, one barrier a step.
__device__ __forceinline__ void moe_tile_product(mf32x4 (&acc)[4][8], const bf16_t* const (&wr)[4],
                                                 const bf16_t* const (&xrow)[2], bf16_t (*s_x)[MOE_TM][MOE_XS], int K) {
    const int lane = threadIdx.x % LLE_WAVE, c = lane / 16, r = lane % 16;
    const int xr = threadIdx.x / 4, xc = 8 * (threadIdx.x % 4);
    mbf16x8 a[4], x0, x1;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) a[nt] = moe_load8(wr[nt], 8 * c, K);
    *(mbf16x8*)&s_x[0][xr][xc] = moe_load8(xrow[0], xc, K);
    *(mbf16x8*)&s_x[0][xr + 64][xc] = moe_load8(xrow[1], xc, K);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += 32, buf ^= 1) {
        mbf16x8 an[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) an[nt] = moe_load8(wr[nt], k0 + 32 + 8 * c, K);
        x0 = moe_load8(xrow[0], k0 + 32 + xc, K);
        x1 = moe_load8(xrow[1], k0 + 32 + xc, K);
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) {
            const mbf16x8 b = *(const mbf16x8*)&s_x[buf][16 * mt + r][8 * c];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt], b, acc[nt][mt], 0, 0, 0);
        }
        *(mbf16x8*)&s_x[buf ^ 1][xr][xc] = x0;  // (read last in the step before, which every wavefront has left)
        *(mbf16x8*)&s_x[buf ^ 1][xr + 64][xc] = x1;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) a[nt] = an[nt];
        __syncthreads();
    }
}

struct MoeTile {
    int expert, row0, rows;  // rows [row0, row0 + rows) of the sorted order, all of `expert`
};

// The tile kernels run on a flat grid of 8 * ceil(tiles * blocks / 8) workgroups.  Workgroups are handed to the
// eight dies in turn, and every die has an L2 of its own: workgroup L works on item (L % 8) * per + L / 8, so that
// a die walks through consecutive items, which are consecutive row tiles (mostly of one expert) against the same
// block of outputs: the tiles that read the same rows of an expert's weights run on one die at about the same time.
__device__ __forceinline__ bool moe_grid_item(int tiles, int blocks, int& tile, int& block) {
    const int per = gridDim.x / 8;
    const int item = (blockIdx.x % 8) * per + blockIdx.x / 8;
    if (item >= tiles * blocks) return false;
    tile = item % tiles;
    block = item / tiles;
    return true;
}

__device__ __forceinline__ bool moe_find_tile(const int32_t* __restrict__ plan, int E, int tile, MoeTile& t) {
    const int32_t* counts = plan;
    const int32_t* first = plan + 2 * E;
    const int32_t* tile0 = plan + 3 * E;
    if (tile >= tile0[E]) return false;
    int e = 0;
    while (tile0[e + 1] <= tile) ++e;
    t.expert = e;
    const int within = (tile - tile0[e]) * MOE_TM;
    t.row0 = first[e] + within;
    t.rows = min(MOE_TM, counts[e] - within);
    return true;
}

// act[row, f] = silu(x Wg^T) * (x Wu^T) for the sorted rows; items (tile, block of 128 f), 4 wavefronts of 32 f each.
// FORM MOE_PLAIN_RELU2: act[row, f] = relu(x Wu^T)^2; items (tile, block of 256 f), 4 wavefronts of 64 f each.
// `in_gains` (or null): a pair's gain as a factor on its products' results, before the activation.
template <int FORM>
__global__ __launch_bounds__(256, 2) void moe_gate_up_tile_kernel(const bf16_t* __restrict__ x,
                                                                const int32_t* __restrict__ plan,
                                                                const int32_t* __restrict__ order,
                                                                const bf16_t* __restrict__ gate_up,
                                                                const float* __restrict__ in_gains,
                                                                bf16_t* __restrict__ act, int E, int top, int F, int K,
                                                                int tiles, int blocks, float limit) {
    MoeTile t;
    int tile, block;
    if (!moe_grid_item(tiles, blocks, tile, block) || !moe_find_tile(plan, E, tile, t)) return;
    __shared__ __attribute__((aligned(16))) bf16_t s_x[2][MOE_TM][MOE_XS];
    const int lane = threadIdx.x % LLE_WAVE, c = lane / 16, r = lane % 16;
    const int per_wave = FORM == MOE_PLAIN_RELU2 ? 64 : 32;
    const int f0 = (block * 4 + threadIdx.x / LLE_WAVE) * per_wave;  // (a wavefront past F multiplies zeros: it shares the barriers)
    const bf16_t* xrow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = threadIdx.x / 4 + 64 * j;
        xrow[j] = row < t.rows ? x + (int64_t)(order[t.row0 + row] / top) * K : nullptr;
    }
    const bf16_t* w = gate_up + (int64_t)t.expert * (FORM == MOE_PLAIN_RELU2 ? 1 : 2) * F * K;
    const bf16_t* wr[4];  // gate rows f0 + r, f0 + 16 + r, then the up rows of the same f; plain: four tiles of up rows
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
        if (FORM == MOE_PLAIN_RELU2) {
            const int f = f0 + nt * 16 + r;
            wr[nt] = f < F ? w + (int64_t)f * K : nullptr;
        } else {
            const int f = f0 + (nt % 2) * 16 + r;
            wr[nt] = f < F ? w + (int64_t)((nt / 2) * F + f) * K : nullptr;
        }
    }
    mf32x4 acc[4][8];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) acc[nt][mt] = mf32x4{0.f, 0.f, 0.f, 0.f};
    moe_tile_product(acc, wr, xrow, s_x, K);
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
        const int row = mt * 16 + r;
        if (row >= t.rows) continue;
        const float gain = in_gains ? in_gains[order[t.row0 + row]] : 1.0f;
        if (FORM == MOE_PLAIN_RELU2) {
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const int f = f0 + nt * 16 + 4 * c;
                if (f >= F) continue;  // (F is a multiple of 4: whole groups)
                mbf16x4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = (bf16_t)moe_relu2(gain * acc[nt][mt][i]);
                *(mbf16x4*)(act + (int64_t)(t.row0 + row) * F + f) = v;
            }
            continue;
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int f = f0 + half * 16 + 4 * c;
            if (f >= F) continue;  // (F is a multiple of 4: whole groups)
            mbf16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float g = gain * acc[half][mt][i], u = gain * acc[2 + half][mt][i];
                v[i] = (bf16_t)moe_gated_act<FORM>(g, u, limit);
            }
            *(mbf16x4*)(act + (int64_t)(t.row0 + row) * F + f) = v;
        }
    }
}

// y[row, o] = act[row] Wd[e]^T for the sorted rows, float32; items (tile, block of 256 o), 4 wavefronts of 64 o each
__global__ __launch_bounds__(256, 2) void moe_down_tile_kernel(const bf16_t* __restrict__ act,
                                                             const int32_t* __restrict__ plan,
                                                             const bf16_t* __restrict__ down, float* __restrict__ y,
                                                             int E, int F, int H, int tiles, int blocks) {
    MoeTile t;
    int tile, block;
    if (!moe_grid_item(tiles, blocks, tile, block) || !moe_find_tile(plan, E, tile, t)) return;
    __shared__ __attribute__((aligned(16))) bf16_t s_x[2][MOE_TM][MOE_XS];
    const int lane = threadIdx.x % LLE_WAVE, c = lane / 16, r = lane % 16;
    const int o0 = (block * 4 + threadIdx.x / LLE_WAVE) * 64;  // (a wavefront past H multiplies zeros: it shares the barriers)
    const bf16_t* xrow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = threadIdx.x / 4 + 64 * j;
        xrow[j] = row < t.rows ? act + (int64_t)(t.row0 + row) * F : nullptr;
    }
    const bf16_t* wr[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
        const int o = o0 + nt * 16 + r;
        wr[nt] = o < H ? down + ((int64_t)t.expert * H + o) * F : nullptr;
    }
    mf32x4 acc[4][8];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) acc[nt][mt] = mf32x4{0.f, 0.f, 0.f, 0.f};
    moe_tile_product(acc, wr, xrow, s_x, F);
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
        const int row = mt * 16 + r;
        if (row >= t.rows) continue;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const int o = o0 + nt * 16 + 4 * c;
            if (o < H) *(mf32x4*)(y + (int64_t)(t.row0 + row) * H + o) = acc[nt][mt];  // (H is a multiple of 4)
        }
    }
}

// out[n, :] = sum_k gains[n, k] * y[place[n top + k], :], in the order of k; a pair without a row (an identity
// expert's) adds its token's own x row
__global__ __launch_bounds__(256) void moe_gather_kernel(const float* __restrict__ y, const int32_t* __restrict__ place,
                                                          const float* __restrict__ gains, const bf16_t* __restrict__ x,
                                                          float* __restrict__ out, int top, int H) {
    const int n = blockIdx.x;
    for (int o = threadIdx.x * 4; o < H; o += blockDim.x * 4) {
        mf32x4 total = mf32x4{0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < top; ++k) {
            const int p = n * top + k;
            const float gain = gains ? gains[p] : 1.0f;  // (no gains: they entered with the experts' inputs)
            if (place[p] < 0) {
                const mbf16x4 xv = *(const mbf16x4*)(x + (int64_t)n * H + o);
                total += gain * mf32x4{(float)xv[0], (float)xv[1], (float)xv[2], (float)xv[3]};
            } else {
                total += gain * *(const mf32x4*)(y + (int64_t)place[p] * H + o);
            }
        }
        *(mf32x4*)(out + (int64_t)n * H + o) = total;
    }
}

extern "C" int lle_moe_tile_rows(void) { return MOE_TM; }

// bfloat16, K and F multiples of 8, H a multiple of 4, E <= 256.  Scratch: plan int32 [4 E + 1], order and
// place int32 [N top], act bfloat16 [N top, F], y float32 [N top, H].
extern "C" int lle_moe_experts_tiled(const void* x, const void* ids, const void* gains, const void* gate_up,
                                     const void* down, void* plan, void* order, void* place, void* act, void* y,
                                     void* out, int N, int top, int E, int F, int K, int H, int form, int gain_on_input,
                                     float limit, hipStream_t stream) {
    if (N <= 0) return 0;
    const int64_t pairs64 = (int64_t)N * top;
    if (top <= 0 || E <= 0 || E > 256 || K % 8 || F % 8 || H % 4 || pairs64 > 0x3fffffff || form < 0 || form > 2)
        return (int)hipErrorInvalidValue;
    const float* in_gains = gain_on_input ? (const float*)gains : nullptr;
    const float* out_gains = gain_on_input ? nullptr : (const float*)gains;
    const int pairs = (int)pairs64;
    const int tiles = pairs / MOE_TM + E;  // at most: every expert leaves one tile partly empty
    moe_zero_kernel<<<(2 * E + 255) / 256, 256, 0, stream>>>((int32_t*)plan, 2 * E);
    moe_count_kernel<<<(pairs + 255) / 256, 256, 0, stream>>>((const int32_t*)ids, (int32_t*)plan, pairs, E);
    moe_plan_kernel<<<1, 256, 0, stream>>>((int32_t*)plan, E);
    moe_place_kernel<<<(pairs + 255) / 256, 256, 0, stream>>>((const int32_t*)ids, (int32_t*)plan, (int32_t*)order,
                                                               (int32_t*)place, pairs, E);
    const int fb = form == MOE_PLAIN_RELU2 ? (F + 255) / 256 : (F + 127) / 128, hb = (H + 255) / 256;
    if (form == MOE_PLAIN_RELU2)
        moe_gate_up_tile_kernel<MOE_PLAIN_RELU2><<<8 * ((tiles * fb + 7) / 8), 256, 0, stream>>>(
            (const bf16_t*)x, (const int32_t*)plan, (const int32_t*)order, (const bf16_t*)gate_up, in_gains, (bf16_t*)act,
            E, top, F, K, tiles, fb, limit);
    else if (form == MOE_GATED_CLAMP)
        moe_gate_up_tile_kernel<MOE_GATED_CLAMP><<<8 * ((tiles * fb + 7) / 8), 256, 0, stream>>>(
            (const bf16_t*)x, (const int32_t*)plan, (const int32_t*)order, (const bf16_t*)gate_up, in_gains, (bf16_t*)act,
            E, top, F, K, tiles, fb, limit);
    else
        moe_gate_up_tile_kernel<MOE_GATED_SILU><<<8 * ((tiles * fb + 7) / 8), 256, 0, stream>>>(
            (const bf16_t*)x, (const int32_t*)plan, (const int32_t*)order, (const bf16_t*)gate_up, in_gains, (bf16_t*)act,
            E, top, F, K, tiles, fb, limit);
    moe_down_tile_kernel<<<8 * ((tiles * hb + 7) / 8), 256, 0, stream>>>(
        (const bf16_t*)act, (const int32_t*)plan, (const bf16_t*)down, (float*)y, E, F, H, tiles, hb);
    moe_gather_kernel<<<N, 256, 0, stream>>>((const float*)y, (const int32_t*)place, out_gains,
                                                (const bf16_t*)x, (float*)out, top, H);
    LLE_RETURN_LAUNCH_STATUS();
}
