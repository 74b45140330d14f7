// Embedding row gather, SiLU-and-mul and the bias of a projection.
// Counterparts in the reference: embedding_forward_kernel
// (src/layers/embedding.cu:91-118) and silu_and_mul_kernel
// (src/ops/silu_and_mul.cu:64-80); both are 32-bit only there.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

// out[n, :] = table[ids[n], :] as 32-bit (the residual stream is 32-bit in
// every mode).  The host has checked 0 <= id < V.
// An id below zero stands for "the token that the last step picked for this token's request": it
// is read from feedback[seq_slots[token_seq[n]]], where the picking kernel left it (a step that
// was launched before the host had read the step before it; the picking kernel only writes ids
// of the vocabulary).
template <typename T>
__global__ __launch_bounds__(256) void embedding_kernel(const int32_t* __restrict__ ids,
                                                         const T* __restrict__ table,
                                                         float* __restrict__ out, int H, float scale,
                                                         const int32_t* __restrict__ feedback,
                                                         const int32_t* __restrict__ token_seq,
                                                         const int32_t* __restrict__ seq_slots) {
    const int64_t n = blockIdx.x;
    int id = ids[n];
    if (id < 0) id = feedback ? feedback[seq_slots[token_seq[n]]] : 0;
    const T* row = table + (int64_t)id * H;
    float* o = out + n * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32<T>(row[i]) * scale;  // (times 1 is exact)
}

// `feedback`, `token_seq` [N] and `seq_slots`: all three or none; every row is multiplied by `scale` in 32-bit
extern "C" int lle_embedding_scaled(const void* ids, const void* table, void* out, int N, int H, int dtype,
                                    const void* feedback, const void* token_seq, const void* seq_slots, float scale,
                                    hipStream_t stream) {
    if (N <= 0) return 0;
    if ((feedback != nullptr) != (token_seq != nullptr) || (feedback != nullptr) != (seq_slots != nullptr))
        return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        embedding_kernel<float><<<N, 256, 0, stream>>>((const int32_t*)ids, (const float*)table, (float*)out, H, scale,
                                                        (const int32_t*)feedback, (const int32_t*)token_seq,
                                                        (const int32_t*)seq_slots);
    else
        embedding_kernel<bf16_t><<<N, 256, 0, stream>>>((const int32_t*)ids, (const bf16_t*)table, (float*)out, H, scale,
                                                         (const int32_t*)feedback, (const int32_t*)token_seq,
                                                         (const int32_t*)seq_slots);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_embedding_feedback(const void* ids, const void* table, void* out, int N, int H, int dtype,
                                      const void* feedback, const void* token_seq, const void* seq_slots,
                                      hipStream_t stream) {
    return lle_embedding_scaled(ids, table, out, N, H, dtype, feedback, token_seq, seq_slots, 1.0f, stream);
}

extern "C" int lle_embedding(const void* ids, const void* table, void* out, int N, int H, int dtype,
                             hipStream_t stream) {
    return lle_embedding_feedback(ids, table, out, N, H, dtype, nullptr, nullptr, nullptr, stream);
}

// gate_up [N, 2I] (gate columns first) -> out [N, I] = gate / (1 + exp(-gate)) * up, in 32-bit
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out,
                                                        int64_t total, int I) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / I;
        const int i = (int)(idx - n * I);
        const float g = to_f32<T>(gate_up[n * 2 * I + i]);
        const float u = to_f32<T>(gate_up[n * 2 * I + I + i]);
        out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
    }
}

// the same for bfloat16 rows whose width is a multiple of 8: 16-byte loads and stores
typedef bf16_t ebf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const bf16_t* __restrict__ gate_up,
                                                            bf16_t* __restrict__ out, int64_t total8, int I8) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / I8;
        const int i = (int)(idx - n * I8);
        const ebf16x8 g = *(const ebf16x8*)(gate_up + (n * 2 * I8 + i) * 8);
        const ebf16x8 u = *(const ebf16x8*)(gate_up + (n * 2 * I8 + I8 + i) * 8);
        ebf16x8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float gf = (float)g[k];
            o[k] = (bf16_t)(gf / (1.0f + expf(-gf)) * (float)u[k]);
        }
        *(ebf16x8*)(out + idx * 8) = o;
    }
}

extern "C" int lle_silu_mul(const void* gate_up, void* out, int N, int I, int dtype, hipStream_t stream) {
    const int64_t total = (int64_t)N * I;
    if (total <= 0) return 0;
    if (dtype == LLE_BF16 && I % 8 == 0) {
        const int64_t total8 = total / 8;
        int64_t vblocks = (total8 + 255) / 256;
        if (vblocks > 16384) vblocks = 16384;
        silu_mul_vec_kernel<<<(int)vblocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, total8, I / 8);
        LLE_RETURN_LAUNCH_STATUS();
    }
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32)
        silu_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, total, I);
    else
        silu_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, total, I);
    LLE_RETURN_LAUNCH_STATUS();
}

// x[m, :] += bias[:] in place, the sum in 32-bit (the reference's Linear has the same optional
// bias, src/layers/linear.cu:169-215; Qwen3 uses none).  `bias` holds TB, x holds T.
template <typename T, typename TB>
__global__ __launch_bounds__(256) void add_bias_kernel(T* __restrict__ x, const TB* __restrict__ bias, int64_t total,
                                                        int N) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        x[idx] = from_f32<T>(to_f32<T>(x[idx]) + to_f32<TB>(bias[idx % N]));
}

extern "C" int lle_add_bias(void* x, const void* bias, int M, int N, int dtype, int bias_dtype, hipStream_t stream) {
    const int64_t total = (int64_t)M * N;
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
#define LLE_BIAS_CASE(T, TB) add_bias_kernel<T, TB><<<(int)blocks, 256, 0, stream>>>((T*)x, (const TB*)bias, total, N)
    if (dtype == LLE_F32 && bias_dtype == LLE_F32) LLE_BIAS_CASE(float, float);
    else if (dtype == LLE_F32) LLE_BIAS_CASE(float, bf16_t);
    else if (bias_dtype == LLE_F32) LLE_BIAS_CASE(bf16_t, float);
    else LLE_BIAS_CASE(bf16_t, bf16_t);
#undef LLE_BIAS_CASE
    LLE_RETURN_LAUNCH_STATUS();
}

// out = x in another float type (the rows of the 32-bit residual stream for a sublayer that reads them)
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void cast_kernel(const TI* __restrict__ x, TO* __restrict__ out, int64_t total) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        out[idx] = from_f32<TO>(to_f32<TI>(x[idx]));
}

extern "C" int lle_cast(const void* x, void* out, int64_t total, int in_dtype, int out_dtype, hipStream_t stream) {
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (in_dtype == LLE_F32 && out_dtype == LLE_BF16)
        cast_kernel<float, bf16_t><<<(int)blocks, 256, 0, stream>>>((const float*)x, (bf16_t*)out, total);
    else if (in_dtype == LLE_BF16 && out_dtype == LLE_F32)
        cast_kernel<bf16_t, float><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)x, (float*)out, total);
    else if (in_dtype == LLE_F32)
        cast_kernel<float, float><<<(int)blocks, 256, 0, stream>>>((const float*)x, (float*)out, total);
    else
        cast_kernel<bf16_t, bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, total);
    LLE_RETURN_LAUNCH_STATUS();
}

// x *= factor in place, float32 (the logits of a model that scales them)
__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ x, int64_t total, float factor) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        x[idx] *= factor;
}

extern "C" int lle_scale(void* x, int64_t total, float factor, hipStream_t stream) {
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    scale_kernel<<<(int)blocks, 256, 0, stream>>>((float*)x, total, factor);
    LLE_RETURN_LAUNCH_STATUS();
}

// out[n, h, :vdim] = a[n, h, :vdim] * sigmoid(gates[n, col0 + h]): a gate per head on an attention's result
// (`a` rows hold heads of D >= vdim elements; what lies past vdim is dropped)
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(const T* __restrict__ a, const T* __restrict__ gates, int gate_cols,
                                                         int col0, T* __restrict__ out, int64_t total, int heads, int D,
                                                         int vdim) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int e = (int)(idx % vdim);
        const int64_t nh = idx / vdim;
        const int h = (int)(nh % heads);
        const int64_t n = nh / heads;
        const float g = to_f32<T>(gates[n * gate_cols + col0 + h]);
        out[idx] = from_f32<T>(to_f32<T>(a[nh * D + e]) / (1.0f + expf(-g)));
    }
}

extern "C" int lle_head_gate(const void* a, const void* gates, int gate_cols, int col0, void* out, int N, int heads, int D,
                             int vdim, int dtype, hipStream_t stream) {
    const int64_t total = (int64_t)N * heads * vdim;
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32)
        head_gate_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)a, (const float*)gates, gate_cols, col0,
                                                                  (float*)out, total, heads, D, vdim);
    else
        head_gate_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)gates, gate_cols, col0,
                                                                   (bf16_t*)out, total, heads, D, vdim);
    LLE_RETURN_LAUNCH_STATUS();
}

// x = tanh(x) in place
template <typename T>
__global__ __launch_bounds__(256) void tanh_kernel(T* __restrict__ x, int64_t total) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        x[idx] = from_f32<T>(tanhf(to_f32<T>(x[idx])));
}

extern "C" int lle_tanh(void* x, int64_t total, int dtype, hipStream_t stream) {
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32) tanh_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)x, total);
    else tanh_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)x, total);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// Activations of feed-forwards that the fused silu product does not cover.
//   gated:  out[n, f] = act(z[n, f] + b[f]) * (z[n, F + f] + b[F + f])        z [N, 2 F]
//   plain:  out[n, f] = act(z[n, f] + b[f])                                   z [N, F]
// times sigmoid(row_gate[n * gate_stride + gate_col]) where a row gate is given (float32).
// act: 0 silu, 1 relu, 2 the square of relu, 3 gelu in its tanh form.  `b` may be null.  Everything in 32-bit.
// ---------------------------------------------------------------------------------
#define LLE_ACT_SILU 0
#define LLE_ACT_RELU 1
#define LLE_ACT_RELU2 2
#define LLE_ACT_GELU_TANH 3

__device__ __forceinline__ float apply_act(float x, int kind) {
    if (kind == LLE_ACT_SILU) return x / (1.0f + expf(-x));
    if (kind == LLE_ACT_GELU_TANH)  // 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))
        return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    const float r = fmaxf(x, 0.f);
    return kind == LLE_ACT_RELU ? r : r * r;
}

template <typename T>
__global__ __launch_bounds__(256) void bias_act_kernel(const T* __restrict__ z, const T* __restrict__ bias,
                                                        const float* __restrict__ row_gate, int gate_stride, int gate_col,
                                                        T* __restrict__ out, int N, int F, int gated, int kind) {
    const int64_t total = (int64_t)N * F;
    const int in_cols = gated ? 2 * F : F;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / F;
        const int f = (int)(idx - n * F);
        const T* row = z + n * in_cols;
        float a = apply_act(to_f32<T>(row[f]) + (bias ? to_f32<T>(bias[f]) : 0.f), kind);
        if (gated) a *= to_f32<T>(row[F + f]) + (bias ? to_f32<T>(bias[F + f]) : 0.f);
        if (row_gate) a *= 1.0f / (1.0f + expf(-row_gate[n * gate_stride + gate_col]));
        out[idx] = from_f32<T>(a);
    }
}

// the same for bfloat16 rows whose width is a multiple of 8: 16-byte loads and stores, eight outputs a thread
template <int GATED, int KIND>
__global__ __launch_bounds__(256) void bias_act_vec_kernel(const bf16_t* __restrict__ z, const bf16_t* __restrict__ bias,
                                                            const float* __restrict__ row_gate, int gate_stride,
                                                            int gate_col, bf16_t* __restrict__ out, int64_t total8,
                                                            int F8) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / F8;
        const int i = (int)(idx - n * F8);
        const int in8 = GATED ? 2 * F8 : F8;
        const ebf16x8 g = *(const ebf16x8*)(z + (n * in8 + i) * 8);
        ebf16x8 u, bg, bu;
        if (GATED) u = *(const ebf16x8*)(z + (n * in8 + F8 + i) * 8);
        if (bias) {
            bg = *(const ebf16x8*)(bias + (int64_t)i * 8);
            if (GATED) bu = *(const ebf16x8*)(bias + (int64_t)(F8 + i) * 8);
        }
        const float rg = row_gate ? 1.0f / (1.0f + expf(-row_gate[n * gate_stride + gate_col])) : 1.0f;
        ebf16x8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            float a = apply_act((float)g[k] + (bias ? (float)bg[k] : 0.f), KIND);
            if (GATED) a *= (float)u[k] + (bias ? (float)bu[k] : 0.f);
            o[k] = (bf16_t)(a * rg);
        }
        *(ebf16x8*)(out + idx * 8) = o;
    }
}

template <int GATED>
static void bias_act_vec(const void* z, const void* bias, const void* row_gate, int gate_stride, int gate_col, void* out,
                         int64_t total8, int F8, int kind, hipStream_t stream) {
    int64_t blocks = (total8 + 255) / 256;
    if (blocks > 16384) blocks = 16384;
#define LLE_ACT_CASE(K)                                                                                              \
    bias_act_vec_kernel<GATED, K><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)z, (const bf16_t*)bias,            \
                                                                    (const float*)row_gate, gate_stride, gate_col,  \
                                                                    (bf16_t*)out, total8, F8)
    if (kind == LLE_ACT_SILU) LLE_ACT_CASE(LLE_ACT_SILU);
    else if (kind == LLE_ACT_RELU) LLE_ACT_CASE(LLE_ACT_RELU);
    else if (kind == LLE_ACT_GELU_TANH) LLE_ACT_CASE(LLE_ACT_GELU_TANH);
    else LLE_ACT_CASE(LLE_ACT_RELU2);
#undef LLE_ACT_CASE
}

extern "C" int lle_bias_act(const void* z, const void* bias, const void* row_gate, int gate_stride, int gate_col,
                            void* out, int N, int F, int gated, int kind, int dtype, hipStream_t stream) {
    if (N <= 0 || F <= 0) return 0;
    if (kind < 0 || kind > LLE_ACT_GELU_TANH) return (int)hipErrorInvalidValue;
    if (dtype == LLE_BF16 && F % 8 == 0) {
        if (gated) bias_act_vec<1>(z, bias, row_gate, gate_stride, gate_col, out, (int64_t)N * F / 8, F / 8, kind, stream);
        else bias_act_vec<0>(z, bias, row_gate, gate_stride, gate_col, out, (int64_t)N * F / 8, F / 8, kind, stream);
        LLE_RETURN_LAUNCH_STATUS();
    }
    int64_t blocks = ((int64_t)N * F + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32)
        bias_act_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)z, (const float*)bias, (const float*)row_gate,
                                                                 gate_stride, gate_col, (float*)out, N, F, gated, kind);
    else
        bias_act_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)z, (const bf16_t*)bias,
                                                                  (const float*)row_gate, gate_stride, gate_col,
                                                                  (bf16_t*)out, N, F, gated, kind);
    LLE_RETURN_LAUNCH_STATUS();
}

// x = cap * tanh(x / cap), float32, in place
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, int64_t total, float cap) {
    const float inv = 1.0f / cap;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        x[idx] = cap * tanhf(x[idx] * inv);
}
extern "C" int lle_softcap(void* x, int64_t total, float cap, hipStream_t stream) {
    if (total <= 0) return 0;
    if (!(cap > 0.f)) return (int)hipErrorInvalidValue;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    softcap_kernel<<<(int)blocks, 256, 0, stream>>>((float*)x, total, cap);
    LLE_RETURN_LAUNCH_STATUS();
}
