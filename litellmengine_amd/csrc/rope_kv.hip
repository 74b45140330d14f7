// Per-head q/k RMSNorm + rotary position encoding + paged K/V write, one launch.
// In the reference these are five reshape copies, two RMSNorm launches, two
// rotary launches and one cudaMemcpy per token and tensor
// (src/model/qwen3.cpp:391-481, src/layers/rotary.cu:153-195,
// src/engine/paged_kv_cache.cpp:138-167).
//
// qkv [N, (nq + 2 nkv) d]: q heads, then k heads, then v heads of one token.
//   q head:  norm over d (weight [d]) -> rotate -> q_out [N, nq, d]
//   k head:  norm over d (weight [d]) -> rotate -> K page of the token's slot
//   v head:  copy                               -> V page of the token's slot
// Rotation pairs element i with i + rot/2 (half split) for i < rot/2; elements
// >= rot pass through.  angle = float(pos) * inv_freq[i], all in 32-bit; cosine and sine of
// every (token, i) are computed once per step by rope_table_kernel ([N][rot/2][2] floats) and
// shared by all heads and all layers.
// A cache page holds K as [nkv][page_size][d] and then V as [nkv][d][page_size]
// (V is kept transposed so that the matrix-core attention kernels find the keys
// of one value column next to each other); slot = page * page_size + offset;
// slot < 0 skips the write.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

template <typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_write_kernel(
    const T* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, int rot, float eps,
    T* __restrict__ q_out, T* __restrict__ kv_layer, int nq, int nkv, int d, int page_size, int64_t page_stride,
    int write_kv) {
    const int64_t n = blockIdx.x;
    const int head = blockIdx.y;  // 0..nq-1 q, then nkv k, then nkv v
    const int lane = threadIdx.x;
    const int width = (nq + 2 * nkv) * d;
    const T* src = qkv + n * width + (int64_t)head * d;

    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    T* dst;
    if (is_q) {
        dst = q_out + (n * nq + head) * d;
    } else {
        if (!write_kv) return;
        const int slot = slots[n];
        if (slot < 0) return;
        const int kvh = is_k ? head - nq : head - nq - nkv;
        const int64_t page = slot / page_size;
        const int off = slot - (int)page * page_size;
        T* page_base = kv_layer + page * page_stride;
        if (!is_k) {  // v: copy into the transposed page, element i of the head at [i][off]
            T* v = page_base + ((int64_t)nkv + kvh) * page_size * d + off;
            for (int i = lane; i < d; i += LLE_WAVE) v[(int64_t)i * page_size] = src[i];
            return;
        }
        dst = page_base + ((int64_t)kvh * page_size + off) * d;
    }

    const void* w = is_q ? q_weight : k_weight;
    float inv = 1.0f;
    if (w) {
        float ss = 0.f;
        for (int i = lane; i < d; i += LLE_WAVE) {
            const float v = to_f32<T>(src[i]);
            ss += v * v;
        }
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)d + eps);
    }
    const int half = rot / 2;
    const float2* cs = (const float2*)cos_sin + n * half;
    for (int i = lane; i < half; i += LLE_WAVE) {
        float x1 = to_f32<T>(src[i]) * inv;
        float x2 = to_f32<T>(src[i + half]) * inv;
        if (w) {
            x1 *= load_as_f32(w, i, weight_dtype);
            x2 *= load_as_f32(w, i + half, weight_dtype);
        }
        const float c = cs[i].x, s = cs[i].y;
        dst[i] = from_f32<T>(x1 * c - x2 * s);
        dst[i + half] = from_f32<T>(x2 * c + x1 * s);
    }
    for (int i = rot + lane; i < d; i += LLE_WAVE) {
        float x = to_f32<T>(src[i]) * inv;
        if (w) x *= load_as_f32(w, i, weight_dtype);
        dst[i] = from_f32<T>(x);
    }
}

// The same for bfloat16 heads of 16, 32, 64, 128 or 256 elements with a rotation over a
// multiple of 16 elements (or none): a lane holds 8 consecutive elements (16-byte loads and
// stores), d / 8 lanes hold a head, a wavefront holds 512 / d heads of one token.  The partner of
// element i in the rotation is i +- rot / 2, which lies rot / 16 lanes away.
typedef bf16_t rbf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void qk_norm_rope_write_vec_kernel(
    const bf16_t* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, int rot, float eps,
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ kv_layer, int nq, int nkv, int d, int page_size,
    int64_t page_stride, int write_kv, int total_heads) {
    // write_kv: 0 = q only, 1 = K and V, 2 = K only (another kernel writes V)
    const int lph = d / 8;  // lanes per head
    const int lane = threadIdx.x % LLE_WAVE;
    const int heads_per_wave = LLE_WAVE / lph;
    const int64_t gw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LLE_WAVE;  // global wavefront
    const int64_t flat = gw * heads_per_wave + lane / lph;                           // (token, head)
    const int hl = lane % lph;                                                        // lane inside the head
    const int per_token = nq + 2 * nkv;
    const bool live = flat < (int64_t)total_heads;
    const int64_t n = live ? flat / per_token : 0;
    const int head = live ? (int)(flat - n * per_token) : 0;
    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    const int e0 = 8 * hl;

    float x[8];
    {
        const rbf16x8 v = *(const rbf16x8*)(qkv + (n * per_token + head) * d + e0);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
    }
    if (is_q || is_k) {
        const void* w = is_q ? q_weight : k_weight;
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, LLE_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * load_as_f32(w, e0 + i, weight_dtype);
        }
        if (rot > 0) {
            const int half = rot / 2;
            const int dl = half / 8;  // lanes between partners
            const bool low = e0 < half, in_rot = e0 < rot;
            float other[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // lanes of the low half read from lane + dl, those of the high half from lane - dl
                const float up = __shfl_down(x[i], dl, LLE_WAVE), down = __shfl_up(x[i], dl, LLE_WAVE);
                other[i] = low ? up : down;
            }
            if (in_rot) {
                // 8 (cos, sin) pairs = four 16-byte loads
                const float4* tab = (const float4*)(cos_sin + (n * half + (low ? e0 : e0 - half)) * 2);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 t = tab[i];  // cos, sin of element 2i, then of 2i + 1
                    x[2 * i] = low ? x[2 * i] * t.x - other[2 * i] * t.y : x[2 * i] * t.x + other[2 * i] * t.y;
                    x[2 * i + 1] = low ? x[2 * i + 1] * t.z - other[2 * i + 1] * t.w
                                       : x[2 * i + 1] * t.z + other[2 * i + 1] * t.w;
                }
            }
        }
    }
    if (!live) return;
    rbf16x8 y;
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (bf16_t)x[i];
    if (is_q) {
        *(rbf16x8*)(q_out + (n * nq + head) * d + e0) = y;
        return;
    }
    if (!write_kv) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int64_t page = slot / page_size;
    const int off = slot - (int)page * page_size;
    bf16_t* page_base = kv_layer + page * page_stride;
    if (is_k) {
        *(rbf16x8*)(page_base + ((int64_t)(head - nq) * page_size + off) * d + e0) = y;
    } else if (write_kv == 1) {
        bf16_t* v = page_base + ((int64_t)nkv + (head - nq - nkv)) * page_size * d + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[(int64_t)(e0 + i) * page_size] = y[i];
    }
}

// The V heads of many tokens into the transposed pages.  A workgroup takes 16 consecutive
// tokens of the batch and one kv head: the rows are read whole into LDS, and every thread
// writes one value element of 8 tokens, as one 16-byte store when those tokens sit in
// consecutive slots of one page starting at a multiple of 8 (prompt portions do), else one by one.
#define VW_TOKENS 16
__device__ __forceinline__ void v_write_transposed_block(const bf16_t* __restrict__ qkv,
                                                         const int32_t* __restrict__ slots,
                                                         bf16_t* __restrict__ kv_layer, int N, int nq, int nkv, int d,
                                                         int page_size, int64_t page_stride, int t0, int kvh,
                                                         bf16_t* tile /* [VW_TOKENS][d + 2] */, int* s_slot) {
    const int width = (nq + 2 * nkv) * d;
    const int row = d + 2;
    for (int idx = threadIdx.x; idx < VW_TOKENS * (d / 8); idx += blockDim.x) {
        const int t = idx / (d / 8), ch = idx % (d / 8);
        if (t0 + t < N) {
            const rbf16x8 v = *(const rbf16x8*)(qkv + (int64_t)(t0 + t) * width + (int64_t)(nq + nkv + kvh) * d + 8 * ch);
#pragma unroll
            for (int i = 0; i < 8; ++i) tile[t * row + 8 * ch + i] = v[i];
        }
    }
    if (threadIdx.x < VW_TOKENS) s_slot[threadIdx.x] = t0 + threadIdx.x < N ? slots[t0 + threadIdx.x] : -1;
    __syncthreads();
    for (int idx = threadIdx.x; idx < 2 * d; idx += blockDim.x) {
        const int g = idx / d, e = idx - g * d;  // tokens 8 g .. 8 g + 7, value element e
        const int first = s_slot[8 * g];
        bool run = first >= 0 && first % 8 == 0 && first % page_size + 8 <= page_size;
#pragma unroll
        for (int i = 1; i < 8; ++i) run = run && s_slot[8 * g + i] == first + i;
        if (run) {
            const int64_t page = first / page_size;
            const int off = first - (int)page * page_size;
            rbf16x8 y;
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = tile[(8 * g + i) * row + e];
            *(rbf16x8*)(kv_layer + page * page_stride + ((int64_t)nkv + kvh) * page_size * d + (int64_t)e * page_size + off) = y;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int slot = s_slot[8 * g + i];
                if (slot < 0) continue;
                const int64_t page = slot / page_size;
                const int off = slot - (int)page * page_size;
                kv_layer[page * page_stride + ((int64_t)nkv + kvh) * page_size * d + (int64_t)e * page_size + off] =
                    tile[(8 * g + i) * row + e];
            }
        }
    }
}
__global__ __launch_bounds__(256) void v_write_transposed_kernel(const bf16_t* __restrict__ qkv,
                                                                  const int32_t* __restrict__ slots,
                                                                  bf16_t* __restrict__ kv_layer, int N, int nq, int nkv,
                                                                  int d, int page_size, int64_t page_stride) {
    extern __shared__ bf16_t tile[];  // [VW_TOKENS][d + 2]
    __shared__ int s_slot[VW_TOKENS];
    v_write_transposed_block(qkv, slots, kv_layer, N, nq, nkv, d, page_size, page_stride, blockIdx.x * VW_TOKENS,
                             blockIdx.y, tile, s_slot);
}

// The same for a rotation over the whole head (rot == d): a lane holds eight elements of the
// low half and their eight partners of the high half (16-byte loads and stores), so the rotation
// needs no exchange between lanes, and one (cos, sin) pair serves both partners.  `per_token`
// heads of a token are this kernel's: q and k, and v too unless the transposing workgroups take it.
__device__ __forceinline__ void load_weights8(const void* w, int e, int dtype, float (&out)[8]) {
    if (dtype == LLE_F32) {
        const float4 a = *(const float4*)((const float*)w + e), b = *(const float4*)((const float*)w + e + 4);
        out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w, out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
    } else {
        const rbf16x8 v = *(const rbf16x8*)((const bf16_t*)w + e);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (float)v[i];
    }
}
__global__ __launch_bounds__(256) void qk_norm_rope_write_pair_kernel(
    const bf16_t* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, float eps,
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ kv_layer, int nq, int nkv, int d, int page_size,
    int64_t page_stride, int write_kv, int64_t total_heads, int per_token, int head_blocks, int N) {
    // write_kv == 2: the workgroups after the first `head_blocks` take the V heads of 16 tokens and
    // one kv head each into the transposed pages (the same launch: the two kinds of work overlap)
    if ((int)blockIdx.x >= head_blocks) {
        extern __shared__ bf16_t tile[];  // [VW_TOKENS][d + 2]
        __shared__ int s_slot[VW_TOKENS];
        const int vb = blockIdx.x - head_blocks;
        v_write_transposed_block(qkv, slots, kv_layer, N, nq, nkv, d, page_size, page_stride, (vb / nkv) * VW_TOKENS,
                                 vb % nkv, tile, s_slot);
        return;
    }
    const int lph = d / 16;  // lanes per head
    const int lane = threadIdx.x % LLE_WAVE;
    const int heads_per_wave = LLE_WAVE / lph;
    const int64_t gw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LLE_WAVE;
    const int64_t flat = gw * heads_per_wave + lane / lph;  // (token, head)
    const int hl = lane % lph;
    const bool live = flat < total_heads;
    const int64_t n = live ? flat / per_token : 0;
    const int head = live ? (int)(flat - n * per_token) : 0;
    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    const int half = d / 2;
    const int e_lo = 8 * hl, e_hi = half + 8 * hl;

    float lo[8], hi[8];
    {
        const bf16_t* src = qkv + (n * (nq + 2 * nkv) + head) * d;
        const rbf16x8 a = *(const rbf16x8*)(src + e_lo), b = *(const rbf16x8*)(src + e_hi);
#pragma unroll
        for (int i = 0; i < 8; ++i) lo[i] = (float)a[i], hi[i] = (float)b[i];
    }
    if (is_q || is_k) {
        // the rotation table is asked for beside the row itself
        const float4* tab = (const float4*)(cos_sin + (n * half + e_lo) * 2);  // (cos, sin) of e_lo .. e_lo + 7
        const float4 t0 = tab[0], t1 = tab[1], t2 = tab[2], t3 = tab[3];
        const void* w = is_q ? q_weight : k_weight;
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += lo[i] * lo[i] + hi[i] * hi[i];
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, LLE_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)d + eps);
            float wl[8], wh[8];
            load_weights8(w, e_lo, weight_dtype, wl);
            load_weights8(w, e_hi, weight_dtype, wh);
#pragma unroll
            for (int i = 0; i < 8; ++i) lo[i] = lo[i] * inv * wl[i], hi[i] = hi[i] * inv * wh[i];
        }
        const float cs[8] = {t0.x, t0.z, t1.x, t1.z, t2.x, t2.z, t3.x, t3.z};
        const float sn[8] = {t0.y, t0.w, t1.y, t1.w, t2.y, t2.w, t3.y, t3.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float a = lo[i], b = hi[i];
            lo[i] = a * cs[i] - b * sn[i];
            hi[i] = b * cs[i] + a * sn[i];
        }
    }
    if (!live) return;
    rbf16x8 ylo, yhi;
#pragma unroll
    for (int i = 0; i < 8; ++i) ylo[i] = (bf16_t)lo[i], yhi[i] = (bf16_t)hi[i];
    if (is_q) {
        bf16_t* dst = q_out + (n * nq + head) * d;
        *(rbf16x8*)(dst + e_lo) = ylo;
        *(rbf16x8*)(dst + e_hi) = yhi;
        return;
    }
    if (!write_kv) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int64_t page = slot / page_size;
    const int off = slot - (int)page * page_size;
    bf16_t* page_base = kv_layer + page * page_stride;
    if (is_k) {
        bf16_t* dst = page_base + ((int64_t)(head - nq) * page_size + off) * d;
        *(rbf16x8*)(dst + e_lo) = ylo;
        *(rbf16x8*)(dst + e_hi) = yhi;
    } else if (write_kv == 1) {
        bf16_t* v = page_base + ((int64_t)nkv + (head - nq - nkv)) * page_size * d + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[(int64_t)(e_lo + i) * page_size] = ylo[i];
            v[(int64_t)(e_hi + i) * page_size] = yhi[i];
        }
    }
}

// cos and sin of float(pos) * inv_freq[i] for every token of the step: out [N][half][2]
__global__ __launch_bounds__(256) void rope_table_kernel(const int32_t* __restrict__ positions,
                                                          const float* __restrict__ inv_freq,
                                                          float* __restrict__ out, int64_t total, int half) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t n = idx / half;
    const int i = (int)(idx - n * half);
    float s, c;
    sincosf((float)positions[n] * inv_freq[i], &s, &c);
    ((float2*)out)[idx] = make_float2(c, s);
}

extern "C" int lle_rope_table(const void* positions, const void* inv_freq, void* out, int N, int half,
                              hipStream_t stream) {
    const int64_t total = (int64_t)N * half;
    if (total <= 0) return 0;
    rope_table_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>((const int32_t*)positions,
                                                                      (const float*)inv_freq, (float*)out, total, half);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_qk_norm_rope_write(const void* qkv, const void* slots,
                                      const void* q_weight, const void* k_weight, int weight_dtype,
                                      const void* cos_sin, int rot, float eps, void* q_out, void* kv_layer,
                                      int N, int nq, int nkv, int d, int page_size, int64_t page_stride,
                                      int write_kv, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    const bool pow2 = d == 16 || d == 32 || d == 64 || d == 128 || d == 256;
    if (dtype == LLE_BF16 && pow2 && rot % 16 == 0 && (int64_t)N * (nq + 2 * nkv) < (1ll << 31)) {
        const int total_heads = N * (nq + 2 * nkv);
        const int heads_per_block = 4 * (LLE_WAVE / (d / 8));
        const int blocks = (total_heads + heads_per_block - 1) / heads_per_block;
        // many tokens: V goes through the transposing kernel (16-byte stores into the pages)
        const bool split_v = write_kv && N >= 64 && page_size % 8 == 0 && (N + VW_TOKENS - 1) / VW_TOKENS <= 0x7fffffff;
        const int64_t v_blocks = split_v ? (int64_t)((N + VW_TOKENS - 1) / VW_TOKENS) * nkv : 0;
        if (rot == d) {
            // the pair kernel: 16 elements a lane; with the transposing workgroups in the same launch
            // the V heads are theirs alone (without a cache write nobody needs them)
            const bool own_v = write_kv && !split_v;
            const int per_token = nq + nkv + (own_v ? nkv : 0);
            const int64_t pair_heads = (int64_t)N * per_token;
            const int pair_heads_per_block = 4 * (LLE_WAVE / (d / 16));
            const int64_t pair_blocks = (pair_heads + pair_heads_per_block - 1) / pair_heads_per_block;
            const bool one_launch = pair_blocks + v_blocks <= 0x7fffffff;
            qk_norm_rope_write_pair_kernel<<<(unsigned)(one_launch ? pair_blocks + v_blocks : pair_blocks), 256,
                                             split_v && one_launch ? VW_TOKENS * (d + 2) * sizeof(bf16_t) : 0, stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, eps,
                (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride,
                write_kv ? (split_v ? 2 : 1) : 0, pair_heads, per_token, (int)pair_blocks, N);
            if (one_launch) LLE_RETURN_LAUNCH_STATUS();
        } else
            qk_norm_rope_write_vec_kernel<<<blocks, 256, 0, stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot,
                eps, (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride,
                write_kv ? (split_v ? 2 : 1) : 0, total_heads);
        if (split_v)
            v_write_transposed_kernel<<<dim3((N + VW_TOKENS - 1) / VW_TOKENS, nkv), 256,
                                        VW_TOKENS * (d + 2) * sizeof(bf16_t), stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, (bf16_t*)kv_layer, N, nq, nkv, d, page_size, page_stride);
        LLE_RETURN_LAUNCH_STATUS();
    }
    dim3 grid(N, nq + 2 * nkv);
    if (dtype == LLE_F32)
        qk_norm_rope_write_kernel<float><<<grid, 64, 0, stream>>>(
            (const float*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot, eps,
            (float*)q_out, (float*)kv_layer, nq, nkv, d, page_size, page_stride, write_kv);
    else
        qk_norm_rope_write_kernel<bf16_t><<<grid, 64, 0, stream>>>(
            (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot, eps,
            (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride, write_kv);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// Projections normed as a whole.  A row of `qkv` holds q [nq dim], then (with keys and values of
// its own) k [nkv dim] and v [nkv vdim], then `extra` columns that are left alone; `bias` (or none)
// covers the whole row.  q and k are divided by the root mean square of their WHOLE projection
// (all heads at once; `per_head`: of each head on its own), times a weight per element (none: times
// one), then the first `rot` elements of every head are rotated in the half-split layout.  The cache's heads hold D >= max(dim, vdim) elements: q leaves
// as [N, nq, D] and K, V^T go to the pages with zeros past dim and vdim.  grid = tokens.
// ---------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float pn_value(const T* __restrict__ row, const T* __restrict__ bias, int e) {
    return to_f32<T>(row[e]) + (bias ? to_f32<T>(bias[e]) : 0.f);
}

// element e (< dim) of head `head` of a projection that starts at column `col0`, normed and rotated
template <typename T>
__device__ __forceinline__ float pn_normed_rotated(const T* __restrict__ row, const T* __restrict__ bias, int col0,
                                                   int head, int dim, int e, float inv, const void* __restrict__ weight,
                                                   int wd, const float* __restrict__ cs, int rot) {
    const int at = head * dim + e;
    const float x = pn_value<T>(row, bias, col0 + at) * inv * (weight ? load_as_f32(weight, at, wd) : 1.0f);
    if (e >= rot) return x;
    const int half = rot / 2;
    const bool low = e < half;
    const int i = low ? e : e - half;
    const int pe = low ? e + half : e - half;
    const float y = pn_value<T>(row, bias, col0 + head * dim + pe) * inv *
                    (weight ? load_as_f32(weight, head * dim + pe, wd) : 1.0f);
    const float c = cs[2 * i], s = cs[2 * i + 1];
    return low ? x * c - y * s : x * c + y * s;
}

#define PN_MAX_HEADS 512  // q heads and kv heads together whose own factors fit the workgroup's LDS

// one factor per head of a projection that starts at column col0: 1 / sqrt(mean of the head's squares + eps)
template <typename T>
__device__ __forceinline__ void pn_head_factors(const T* __restrict__ row, const T* __restrict__ bias, int col0, int heads,
                                                int dim, float eps, float* __restrict__ inv) {
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE, waves = blockDim.x / LLE_WAVE;
    for (int h = wave; h < heads; h += waves) {
        float ss = 0.f;
        for (int e = lane; e < dim; e += LLE_WAVE) {
            const float x = pn_value<T>(row, bias, col0 + h * dim + e);
            ss += x * x;
        }
        ss = wave_sum(ss);
        if (lane == 0) inv[h] = 1.0f / sqrtf(ss / (float)dim + eps);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void proj_norm_rope_write_kernel(
    const T* __restrict__ qkv, int cols, const T* __restrict__ bias, const int32_t* __restrict__ slots,
    const void* __restrict__ q_weight, const void* __restrict__ k_weight, int wd, const float* __restrict__ cos_sin,
    int rot, float eps, T* __restrict__ q_out, T* __restrict__ kv_layer, int nq, int nkv, int dim, int vdim, int D,
    int page_size, int64_t page_stride, int has_kv, int write_kv, int per_head) {
    __shared__ float red[16];
    __shared__ float head_inv[PN_MAX_HEADS];
    const int64_t n = blockIdx.x;
    const T* row = qkv + n * cols;
    const float* cs = cos_sin + n * rot;  // [rot / 2][2]
    const int qw = nq * dim, kw = nkv * dim;
    float inv_q = 0.f, inv_k = 0.f;
    if (per_head) {
        pn_head_factors<T>(row, bias, 0, nq, dim, eps, head_inv);
        if (has_kv) pn_head_factors<T>(row, bias, qw, nkv, dim, eps, head_inv + nq);
        __syncthreads();
    } else {
        float ss = 0.f;
        for (int e = threadIdx.x; e < qw; e += blockDim.x) {
            const float x = pn_value<T>(row, bias, e);
            ss += x * x;
        }
        inv_q = 1.0f / sqrtf(block_sum(ss, red) / (float)qw + eps);
    }
    for (int idx = threadIdx.x; idx < nq * D; idx += blockDim.x) {
        const int h = idx / D, e = idx - h * D;
        const float inv = per_head ? head_inv[h] : inv_q;
        const float y = e < dim ? pn_normed_rotated<T>(row, bias, 0, h, dim, e, inv, q_weight, wd, cs, rot) : 0.f;
        q_out[n * nq * D + idx] = from_f32<T>(y);
    }
    if (!has_kv) return;
    if (!per_head) {
        float ss = 0.f;
        for (int e = threadIdx.x; e < kw; e += blockDim.x) {
            const float x = pn_value<T>(row, bias, qw + e);
            ss += x * x;
        }
        inv_k = 1.0f / sqrtf(block_sum(ss, red) / (float)kw + eps);
    }
    const int slot = slots[n];
    if (!write_kv || slot < 0) return;
    const int page = slot / page_size, off = slot - page * page_size;
    T* dst = kv_layer + (int64_t)page * page_stride;
    for (int idx = threadIdx.x; idx < nkv * D; idx += blockDim.x) {
        const int h = idx / D, e = idx - h * D;
        const float inv = per_head ? head_inv[nq + h] : inv_k;
        const float y = e < dim ? pn_normed_rotated<T>(row, bias, qw, h, dim, e, inv, k_weight, wd, cs, rot) : 0.f;
        dst[((int64_t)h * page_size + off) * D + e] = from_f32<T>(y);
        const float v = e < vdim ? pn_value<T>(row, bias, qw + kw + h * vdim + e) : 0.f;
        dst[(int64_t)nkv * page_size * D + ((int64_t)h * D + e) * page_size + off] = from_f32<T>(v);
    }
}

extern "C" int lle_proj_norm_rope_write(const void* qkv, int cols, const void* bias, const void* slots,
                                        const void* q_weight, const void* k_weight, int weight_dtype, const void* cos_sin,
                                        int rot, float eps, void* q_out, void* kv_layer, int N, int nq, int nkv, int dim,
                                        int vdim, int D, int page_size, int64_t page_stride, int has_kv, int write_kv,
                                        int per_head, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (rot % 2 || rot > dim || dim > D || vdim > D || (rot > 0 && cos_sin == nullptr)) return (int)hipErrorInvalidValue;
    if (per_head && nq + nkv > PN_MAX_HEADS) return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        proj_norm_rope_write_kernel<float><<<N, 256, 0, stream>>>(
            (const float*)qkv, cols, (const float*)bias, (const int32_t*)slots, q_weight, k_weight, weight_dtype,
            (const float*)cos_sin, rot, eps, (float*)q_out, (float*)kv_layer, nq, nkv, dim, vdim, D, page_size, page_stride,
            has_kv, write_kv, per_head);
    else
        proj_norm_rope_write_kernel<bf16_t><<<N, 256, 0, stream>>>(
            (const bf16_t*)qkv, cols, (const bf16_t*)bias, (const int32_t*)slots, q_weight, k_weight, weight_dtype,
            (const float*)cos_sin, rot, eps, (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, dim, vdim, D, page_size,
            page_stride, has_kv, write_kv, per_head);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// Projections behind a short causal convolution over time.  A row of `u` holds q [nq dim], k [nkv dim]
// and v [nkv vdim] of one token.  Per channel c and token t of a request,
//     conv_t[c] = sum_j taps[c, j] * u_(t - J + 1 + j)[c]          taps float32 [cols, J]
// where a row before the portion that this step brings comes from the request's state row (the last
// J - 1 rows of u of the steps before, oldest first, float32; zeros at a request's start) and rows before
// the request's start are zeros by that.  Then every head of q and k is divided by its root mean square
// times one weight [dim] for all heads, the first `rot` elements of every head are rotated in the half-split
// layout, q leaves as [N, nq, D] (zeros past dim) and K, V^T go to the pages with zeros past dim and vdim.
// grid = tokens, a wavefront of the workgroup per head, four heads at a time; all arithmetic in 32-bit.
// The state is advanced by conv_state_kernel, a launch of its own behind this one (every token of a
// portion reads the rows that the step found there).
// ---------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float conv_at(const T* __restrict__ u, int cols, const float* __restrict__ taps, int J,
                                         const float* __restrict__ kept, int64_t n, int before, int c) {
    // `before`: rows of this request in this step ahead of row n; kept: [J - 1, cols] or null
    float acc = 0.f;
    for (int j = 0; j < J; ++j) {
        const int back = J - 1 - j;  // how many tokens back this tap reaches
        float x;
        if (back <= before)
            x = to_f32<T>(u[(n - back) * cols + c]);
        else
            x = kept ? kept[(int64_t)(J - 1 - (back - before)) * cols + c] : 0.f;
        acc += taps[(int64_t)c * J + j] * x;
    }
    return acc;
}

template <typename T>
__global__ __launch_bounds__(256) void conv_norm_rope_write_kernel(
    const T* __restrict__ u, int cols, const float* __restrict__ taps, int J, const float* __restrict__ state,
    int64_t state_stride, const int32_t* __restrict__ token_seq, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ slots, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos_sin, int rot, float eps, T* __restrict__ q_out,
    T* __restrict__ kv_layer, int nq, int nkv, int dim, int vdim, int D, int page_size, int64_t page_stride,
    int write_kv) {
    extern __shared__ float conv_row[];  // the token's convolved q and k heads, one head per wavefront at a time
    const int64_t n = blockIdx.x;
    const int seq = token_seq[n];
    const int before = (int)(n - cu_tokens[seq]);
    const float* kept = (state && J > 1) ? state + (int64_t)seq_slots[seq] * state_stride : nullptr;
    const float* cs = cos_sin + n * rot;  // [rot / 2][2]
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE, waves = blockDim.x / LLE_WAVE;
    float* mine = conv_row + (int64_t)wave * dim;
    const int slot = slots[n];
    const bool writes = write_kv && slot >= 0;
    const int page = writes ? slot / page_size : 0, off = writes ? slot - page * page_size : 0;
    T* dst = kv_layer + (int64_t)page * page_stride;
    const int half = rot / 2;
    const int heads = nq + (writes ? nkv : 0);
    for (int h0 = 0; h0 < heads; h0 += waves) {  // (the same number of rounds for every wavefront: barriers inside)
        const int h = h0 + wave;
        const bool active = h < heads;
        const bool is_q = h < nq;
        const int col0 = is_q ? h * dim : nq * dim + (h - nq) * dim;
        const float* w = is_q ? q_weight : k_weight;
        float ss = 0.f;
        if (active)
            for (int e = lane; e < dim; e += LLE_WAVE) {
                const float x = conv_at<T>(u, cols, taps, J, kept, n, before, col0 + e);
                mine[e] = x;
                ss += x * x;
            }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
        __syncthreads();
        if (active)
            for (int e = lane; e < D; e += LLE_WAVE) {
                float y = 0.f;
                if (e < dim) {
                    y = mine[e] * inv * w[e];
                    if (e < rot) {
                        const bool low = e < half;
                        const int i = low ? e : e - half;
                        const int pe = low ? e + half : e - half;
                        const float p = mine[pe] * inv * w[pe];
                        const float c = cs[2 * i], s = cs[2 * i + 1];
                        y = low ? y * c - p * s : y * c + p * s;
                    }
                }
                if (is_q)
                    q_out[(n * nq + h) * D + e] = from_f32<T>(y);
                else
                    dst[((int64_t)(h - nq) * page_size + off) * D + e] = from_f32<T>(y);
            }
        __syncthreads();
    }
    if (!writes) return;
    const int v0 = (nq + nkv) * dim;
    for (int idx = threadIdx.x; idx < nkv * D; idx += blockDim.x) {
        const int h = idx / D, e = idx - h * D;
        const float v = e < vdim ? conv_at<T>(u, cols, taps, J, kept, n, before, v0 + h * vdim + e) : 0.f;
        dst[(int64_t)nkv * page_size * D + ((int64_t)h * D + e) * page_size + off] = from_f32<T>(v);
    }
}

// The same for up to CV_MAX_TAPS taps and heads of up to 64 CV_ITEMS elements, which is what models have: a
// wavefront per (head, run of `tile` consecutive tokens), grid (token tiles, heads / 4); the v part of a row
// counts as heads of its own (no norm, no rotation).  A lane owns up to CV_ITEMS items of its head, an item being
// a rotated pair (element i and i + rot / 2) or one element past the rotation: the partner of a rotation sits in
// the same lane, the norm's sum crosses the lanes once, nothing passes through LDS and no barrier is met.  The
// lane keeps its channels' taps and the last J - 1 values of u in registers and walks its tokens in order: while
// the request stays the same a token costs one new load per channel, whatever J.
#define CV_MAX_TAPS 8
#define CV_ITEMS 4

template <typename T, int J>
__global__ __launch_bounds__(256) void conv_norm_rope_write_tile_kernel(
    const T* __restrict__ u, int cols, const float* __restrict__ taps, const float* __restrict__ state,
    int64_t state_stride, const int32_t* __restrict__ token_seq, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ slots, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos_sin, int rot, float eps, T* __restrict__ q_out,
    T* __restrict__ kv_layer, int N, int nq, int nkv, int dim, int vdim, int D, int page_size, int64_t page_stride,
    int write_kv, int tile) {
    constexpr int W = J > 1 ? J - 1 : 1;
    const int lane = threadIdx.x % LLE_WAVE;
    const int h = blockIdx.y * (blockDim.x / LLE_WAVE) + threadIdx.x / LLE_WAVE;
    if (h >= nq + (write_kv ? 2 * nkv : 0)) return;  // (the whole wavefront; no barrier follows)
    const bool is_q = h < nq, is_v = h >= nq + nkv;
    const int width = is_v ? vdim : dim;
    const int hrot = is_v ? 0 : rot, half = hrot / 2;
    const int items = half + (width - hrot);
    const int col0 = is_q ? h * dim : is_v ? (nq + nkv) * dim + (h - nq - nkv) * vdim : nq * dim + (h - nq) * dim;
    const float* nw = is_q ? q_weight : k_weight;
    int ca[CV_ITEMS], cb[CV_ITEMS];  // the item's elements of the head (cb < 0: no partner)
    float ta[CV_ITEMS][J], tb[CV_ITEMS][J], wa[CV_ITEMS], wb[CV_ITEMS], xa[CV_ITEMS][W], xb[CV_ITEMS][W];
#pragma unroll
    for (int i = 0; i < CV_ITEMS; ++i) {
        const int it = lane + LLE_WAVE * i;
        ca[i] = it < half ? it : hrot + (it - half);
        cb[i] = it < half ? it + half : -1;
        if (it >= items) ca[i] = -1;
        wa[i] = wb[i] = 1.f;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            ta[i][j] = ca[i] >= 0 ? taps[(int64_t)(col0 + ca[i]) * J + j] : 0.f;
            tb[i][j] = (ca[i] >= 0 && cb[i] >= 0) ? taps[(int64_t)(col0 + cb[i]) * J + j] : 0.f;
        }
        if (!is_v && ca[i] >= 0) {
            wa[i] = nw[ca[i]];
            if (cb[i] >= 0) wb[i] = nw[cb[i]];
        }
#pragma unroll
        for (int j = 0; j < W; ++j) xa[i][j] = xb[i][j] = 0.f;
    }
    const int64_t n0 = (int64_t)blockIdx.x * tile;
    int prev_seq = -1;
    for (int tk = 0; tk < tile; ++tk) {
        const int64_t n = n0 + tk;
        if (n >= N) break;
        const int seq = token_seq[n];
        float va[CV_ITEMS], vb[CV_ITEMS];
        if (seq != prev_seq && J > 1) {  // the first token of this wavefront's run, or another request: fill the window
            const int before = (int)(n - cu_tokens[seq]);
            const float* kept = state ? state + (int64_t)seq_slots[seq] * state_stride : nullptr;
#pragma unroll
            for (int j = 0; j < W; ++j) {
                const int back = J - 1 - j;
#pragma unroll
                for (int i = 0; i < CV_ITEMS; ++i) {
                    float a = 0.f, b = 0.f;
                    if (ca[i] >= 0) {
                        if (back <= before) {
                            a = to_f32<T>(u[(n - back) * cols + col0 + ca[i]]);
                            if (cb[i] >= 0) b = to_f32<T>(u[(n - back) * cols + col0 + cb[i]]);
                        } else if (kept) {
                            const int64_t r = (int64_t)(J - 1 - (back - before)) * cols + col0;
                            a = kept[r + ca[i]];
                            if (cb[i] >= 0) b = kept[r + cb[i]];
                        }
                    }
                    xa[i][j] = a;
                    xb[i][j] = b;
                }
            }
        }
        prev_seq = seq;
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CV_ITEMS; ++i) {
            float a = 0.f, b = 0.f;
            if (ca[i] >= 0) {
                a = to_f32<T>(u[n * cols + col0 + ca[i]]);
                if (cb[i] >= 0) b = to_f32<T>(u[n * cols + col0 + cb[i]]);
            }
            float sa = ta[i][J - 1] * a, sb = tb[i][J - 1] * b;
#pragma unroll
            for (int j = 0; j < J - 1; ++j) {
                sa += ta[i][j] * xa[i][j];
                sb += tb[i][j] * xb[i][j];
            }
#pragma unroll
            for (int j = 0; j + 1 < J - 1; ++j) {  // the window moves on by one token
                xa[i][j] = xa[i][j + 1];
                xb[i][j] = xb[i][j + 1];
            }
            if (J > 1) {
                xa[i][W - 1] = a;
                xb[i][W - 1] = b;
            }
            va[i] = sa;
            vb[i] = sb;
            ss += sa * sa + sb * sb;
        }
        const int slot = slots[n];
        const bool writes = is_q || slot >= 0;
        const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - page * page_size : 0;
        T* dst = kv_layer + (int64_t)page * page_stride;
        if (is_v) {
            if (!writes) continue;
            T* vt = dst + (int64_t)nkv * page_size * D + (int64_t)(h - nq - nkv) * D * page_size + off;
#pragma unroll
            for (int i = 0; i < CV_ITEMS; ++i)
                if (ca[i] >= 0) vt[(int64_t)ca[i] * page_size] = from_f32<T>(va[i]);
            for (int e = vdim + lane; e < D; e += LLE_WAVE) vt[(int64_t)e * page_size] = from_f32<T>(0.f);
            continue;
        }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
        if (!writes) continue;
        T* row = is_q ? q_out + (n * nq + h) * D : dst + ((int64_t)(h - nq) * page_size + off) * D;
        const float* cs = cos_sin + n * rot;  // [rot / 2][2]
#pragma unroll
        for (int i = 0; i < CV_ITEMS; ++i) {
            if (ca[i] < 0) continue;
            const float a = va[i] * inv * wa[i];
            if (cb[i] >= 0) {
                const float b = vb[i] * inv * wb[i];
                const float c = cs[2 * ca[i]], sn = cs[2 * ca[i] + 1];
                row[ca[i]] = from_f32<T>(a * c - b * sn);
                row[cb[i]] = from_f32<T>(b * c + a * sn);
            } else {
                row[ca[i]] = from_f32<T>(a);
            }
        }
        for (int e = dim + lane; e < D; e += LLE_WAVE) row[e] = from_f32<T>(0.f);
    }
}

template <typename T>
static bool conv_tile_launch(int J, dim3 grid, hipStream_t stream, const void* u, int cols, const void* taps,
                             const void* state, int64_t state_stride, const void* token_seq, const void* cu_tokens,
                             const void* seq_slots, const void* slots, const void* q_weight, const void* k_weight,
                             const void* cos_sin, int rot, float eps, void* q_out, void* kv_layer, int N, int nq, int nkv,
                             int dim, int vdim, int D, int page_size, int64_t page_stride, int write_kv, int tile) {
#define LLE_CONV_CASE(JJ)                                                                                               \
    case JJ:                                                                                                            \
        conv_norm_rope_write_tile_kernel<T, JJ><<<grid, 256, 0, stream>>>(                                              \
            (const T*)u, cols, (const float*)taps, (const float*)state, state_stride, (const int32_t*)token_seq,        \
            (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (const int32_t*)slots, (const float*)q_weight,        \
            (const float*)k_weight, (const float*)cos_sin, rot, eps, (T*)q_out, (T*)kv_layer, N, nq, nkv, dim, vdim, D, \
            page_size, page_stride, write_kv, tile);                                                                    \
        return true;
    switch (J) {
        LLE_CONV_CASE(1)
        LLE_CONV_CASE(2)
        LLE_CONV_CASE(3)
        LLE_CONV_CASE(4)
        LLE_CONV_CASE(5)
        LLE_CONV_CASE(6)
        LLE_CONV_CASE(7)
        LLE_CONV_CASE(8)
    }
#undef LLE_CONV_CASE
    return false;
}

// state row of every request of the step <- the last `kept` rows of (what it held, then the step's rows of u)
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ u, int cols, float* __restrict__ state,
                                                          int64_t state_stride, int kept,
                                                          const int32_t* __restrict__ cu_tokens,
                                                          const int32_t* __restrict__ seq_slots) {
    const int seq = blockIdx.y;
    const int q0 = cu_tokens[seq], L = cu_tokens[seq + 1] - q0;
    if (L <= 0) return;
    float* row = state + (int64_t)seq_slots[seq] * state_stride;
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < cols; c += gridDim.x * blockDim.x) {
        for (int r = 0; r < kept; ++r) {  // (r rises: a row is read before a thread of this channel overwrites it)
            const int src = L + r;  // index into [kept old rows | L new rows]
            row[(int64_t)r * cols + c] = src < kept ? row[(int64_t)src * cols + c]
                                                    : to_f32<T>(u[(int64_t)(q0 + src - kept) * cols + c]);
        }
    }
}

extern "C" int lle_conv_norm_rope_write(const void* u, int cols, const void* taps, int J, const void* state,
                                        int64_t state_stride, const void* token_seq, const void* cu_tokens,
                                        const void* seq_slots, const void* slots, const void* q_weight,
                                        const void* k_weight, const void* cos_sin, int rot, float eps, void* q_out,
                                        void* kv_layer, int N, int nq, int nkv, int dim, int vdim, int D, int page_size,
                                        int64_t page_stride, int write_kv, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (J < 1 || rot % 2 || rot > dim || dim > D || vdim > D || (rot > 0 && cos_sin == nullptr) ||
        cols < (nq + nkv) * dim + nkv * vdim)
        return (int)hipErrorInvalidValue;
    if (J <= CV_MAX_TAPS && dim <= CV_ITEMS * LLE_WAVE && vdim <= CV_ITEMS * LLE_WAVE) {
        // runs of tokens long enough that the taps are loaded seldom, short enough that a prompt fills the chip
        // (measured at 2048 tokens: runs of 16 tokens where that leaves some 768 workgroups, shorter runs otherwise)
        const int heads = nq + (write_kv ? 2 * nkv : 0);
        const int64_t fit = (int64_t)N * ((heads + 3) / 4) / 768;
        const int tile = fit >= 16 ? 16 : fit >= 8 ? 8 : fit >= 4 ? 4 : fit >= 2 ? 2 : 1;
        const dim3 grid((N + tile - 1) / tile, (heads + 3) / 4);
        if (grid.y <= 65535) {
            if (dtype == LLE_F32)
                conv_tile_launch<float>(J, grid, stream, u, cols, taps, state, state_stride, token_seq, cu_tokens, seq_slots,
                                        slots, q_weight, k_weight, cos_sin, rot, eps, q_out, kv_layer, N, nq, nkv, dim, vdim,
                                        D, page_size, page_stride, write_kv, tile);
            else
                conv_tile_launch<bf16_t>(J, grid, stream, u, cols, taps, state, state_stride, token_seq, cu_tokens,
                                         seq_slots, slots, q_weight, k_weight, cos_sin, rot, eps, q_out, kv_layer, N, nq, nkv,
                                         dim, vdim, D, page_size, page_stride, write_kv, tile);
            LLE_RETURN_LAUNCH_STATUS();
        }
    }
    const size_t lds = (size_t)4 * dim * sizeof(float);
    if (dtype == LLE_F32)
        conv_norm_rope_write_kernel<float><<<N, 256, lds, stream>>>(
            (const float*)u, cols, (const float*)taps, J, (const float*)state, state_stride, (const int32_t*)token_seq,
            (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (const int32_t*)slots, (const float*)q_weight,
            (const float*)k_weight, (const float*)cos_sin, rot, eps, (float*)q_out, (float*)kv_layer, nq, nkv, dim, vdim, D,
            page_size, page_stride, write_kv);
    else
        conv_norm_rope_write_kernel<bf16_t><<<N, 256, lds, stream>>>(
            (const bf16_t*)u, cols, (const float*)taps, J, (const float*)state, state_stride, (const int32_t*)token_seq,
            (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (const int32_t*)slots, (const float*)q_weight,
            (const float*)k_weight, (const float*)cos_sin, rot, eps, (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, dim, vdim,
            D, page_size, page_stride, write_kv);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_conv_state_update(const void* u, int cols, void* state, int64_t state_stride, int kept,
                                     const void* cu_tokens, const void* seq_slots, int S, int dtype,
                                     hipStream_t stream) {
    if (S <= 0 || kept <= 0) return 0;
    if (S > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid((cols + 255) / 256, S);
    if (dtype == LLE_F32)
        conv_state_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, cols, (float*)state, state_stride, kept,
                                                            (const int32_t*)cu_tokens, (const int32_t*)seq_slots);
    else
        conv_state_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, cols, (float*)state, state_stride, kept,
                                                             (const int32_t*)cu_tokens, (const int32_t*)seq_slots);
    LLE_RETURN_LAUNCH_STATUS();
}
