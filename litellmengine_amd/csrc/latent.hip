// Latent attention: the cache holds, per token, one latent row c [rank] and one rotated key part
// k_rot [rot] shared by all heads; a page is [page_size][rank] of c, then the same latents
// transposed, [rank][page_size] (the matrix cores contract over keys in the second product and
// want the keys of one element side by side), then [page_size][rot] of k_rot.  Queries arrive already carried into the latent space
// (q_lat [N, H, rank], float32 or the cache's type) together with their rotated part
// (q_rot [N, H, rot], float32), so all heads of a token attend to the same rows:
//   score_j = (q_lat . c_j + q_rot . k_rot_j) * scale
//   p = softmax over the visible keys and one sink per head (exp(sink) in the denominator, no value)
//   o_lat = sum_j p_j c_j                 [N, H, rank]
// Scores, softmax and sums are 32-bit.  Rotation: neighbouring pairs (2i, 2i + 1).
#include "common.h"

LLE_DEFINE_ERROR_STRING()

// ---------------------------------------------------------------------------------------------
// dkv [N, rank + rot] -> c = RMSNorm(dkv[:rank]) * w, k_rot = rotate(dkv[rank:]) into the pages
// at slots[n] (page = slot / P, place = slot % P; slot < 0: nothing is written).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ dkv,
                                                               const void* __restrict__ norm_w, int w_dtype,
                                                               float eps, const float* __restrict__ cos_sin,
                                                               int rot_dims, const int32_t* __restrict__ slots,
                                                               T* __restrict__ pages, int64_t page_stride, int P,
                                                               int rank, int rot) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const int slot = slots[n];
    if (slot < 0) return;  // (the whole workgroup)
    const T* row = dkv + n * (rank + rot);
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
        const float v = to_f32<T>(row[i]);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
    T* page = pages + (int64_t)(slot / P) * page_stride;
    T* c = page + (int64_t)(slot % P) * rank;
    T* ct = page + (int64_t)P * rank + (slot % P);
    T* kr = page + (int64_t)2 * P * rank + (int64_t)(slot % P) * rot;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
        const T v = from_f32<T>(to_f32<T>(row[i]) * inv * load_as_f32(norm_w, i, w_dtype));
        c[i] = v;
        ct[(int64_t)i * P] = v;
    }
    const float* cs = cos_sin + n * rot_dims;  // [rot_dims / 2][2]
    for (int i = threadIdx.x; i < rot; i += blockDim.x) {
        float v = to_f32<T>(row[rank + i]);
        if (i < rot_dims) {
            const float co = cs[(i >> 1) * 2], si = cs[(i >> 1) * 2 + 1];
            const float other = to_f32<T>(row[rank + (i ^ 1)]);
            v = (i & 1) ? v * co + other * si : v * co - other * si;
        }
        kr[i] = from_f32<T>(v);
    }
}

extern "C" int lle_latent_kv_write(const void* dkv, const void* norm_w, int w_dtype, float eps, const void* cos_sin,
                                   int rot_dims, const void* slots, void* pages, int64_t page_stride, int P, int N,
                                   int rank, int rot, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (rot_dims < 0 || rot_dims > rot || rot_dims % 2 || (rot_dims > 0 && cos_sin == nullptr) || P <= 0)
        return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        latent_kv_write_kernel<float><<<N, 256, 0, stream>>>((const float*)dkv, norm_w, w_dtype, eps,
                                                              (const float*)cos_sin, rot_dims, (const int32_t*)slots,
                                                              (float*)pages, page_stride, P, rank, rot);
    else
        latent_kv_write_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)dkv, norm_w, w_dtype, eps,
                                                               (const float*)cos_sin, rot_dims, (const int32_t*)slots,
                                                               (bf16_t*)pages, page_stride, P, rank, rot);
    LLE_RETURN_LAUNCH_STATUS();
}

// q [N, H, dim + rot] -> the rotated parts, float32 [N, H, rot]
template <typename T>
__global__ __launch_bounds__(256) void latent_q_rope_kernel(const T* __restrict__ q, const float* __restrict__ cos_sin,
                                                             int rot_dims, float* __restrict__ out, int64_t total,
                                                             int H, int dim, int rot) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(idx % rot);
        const int64_t nh = idx / rot;
        const int64_t n = nh / H;
        const T* src = q + nh * (dim + rot) + dim;
        float v = to_f32<T>(src[i]);
        if (i < rot_dims) {
            const float* cs = cos_sin + n * rot_dims;
            const float co = cs[(i >> 1) * 2], si = cs[(i >> 1) * 2 + 1];
            const float other = to_f32<T>(src[i ^ 1]);
            v = (i & 1) ? v * co + other * si : v * co - other * si;
        }
        out[idx] = v;
    }
}

extern "C" int lle_latent_q_rope(const void* q, const void* cos_sin, int rot_dims, void* out, int N, int H, int dim,
                                 int rot, int dtype, hipStream_t stream) {
    const int64_t total = (int64_t)N * H * rot;
    if (total <= 0) return 0;
    if (rot_dims < 0 || rot_dims > rot || rot_dims % 2 || (rot_dims > 0 && cos_sin == nullptr))
        return (int)hipErrorInvalidValue;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32)
        latent_q_rope_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)q, (const float*)cos_sin, rot_dims,
                                                                      (float*)out, total, H, dim, rot);
    else
        latent_q_rope_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)q, (const float*)cos_sin, rot_dims,
                                                                       (float*)out, total, H, dim, rot);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// The attention for any sizes and either type: one workgroup per (token, head).  The keys are
// walked 256 at a time: thread j takes the score of key j (both dot products, the query in LDS),
// the workgroup rescales its running maximum and sum (which start at the sink: m = sink, l = 1),
// then thread r adds the 256 weighted rows into element r of the result.
// ---------------------------------------------------------------------------------------------
#define LAT_TILE 256
#define LAT_MAX_RANK_PER_THREAD 4  // rank <= 1024

template <typename T, typename TQ>
__global__ __launch_bounds__(LAT_TILE) void latent_attention_generic_kernel(
    const TQ* __restrict__ q_lat, int64_t ql_stride_n, int64_t ql_stride_h, const float* __restrict__ q_rot,
    const T* __restrict__ pages, int64_t page_stride, int P, int rank, int rot,
    const int32_t* __restrict__ block_table, int max_pages, const int32_t* __restrict__ seq_slots,
    const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ kv_lens,
    const int32_t* __restrict__ token_seq, const float* __restrict__ sink, int window, float scale,
    T* __restrict__ out, int H) {
    extern __shared__ int64_t lds[];
    int64_t* where = (int64_t*)lds;          // [LAT_TILE] offset of every key's c row in `pages`
    float* pw = (float*)(where + LAT_TILE);  // [LAT_TILE] weights of the tile's keys
    float* red = pw + LAT_TILE;              // [16]
    float* qa = red + 16;                    // [rank]
    float* qr = qa + rank;                   // [rot]

    const int n = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int s = token_seq[n];
    const int q0 = cu_tokens[s], q_len = cu_tokens[s + 1] - q0;
    const int pos = kv_lens[s] - q_len + (n - q0);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int32_t* table = block_table + (int64_t)seq_slots[s] * max_pages;

    const TQ* ql = q_lat + n * ql_stride_n + h * ql_stride_h;
    for (int i = tid; i < rank; i += LAT_TILE) qa[i] = to_f32<TQ>(ql[i]);
    const float* qrs = q_rot + ((int64_t)n * H + h) * rot;
    for (int i = tid; i < rot; i += LAT_TILE) qr[i] = qrs[i];
    __syncthreads();

    // the sink: a key with score `sink` and no value; without one the sum starts empty (the first tile holds
    // the token itself, so the maximum is finite from there on)
    float m = sink ? sink[h] : -INFINITY, l = sink ? 1.0f : 0.0f;
    float acc[LAT_MAX_RANK_PER_THREAD];
#pragma unroll
    for (int k = 0; k < LAT_MAX_RANK_PER_THREAD; ++k) acc[k] = 0.f;

    for (int base = lo; base <= pos; base += LAT_TILE) {
        const int j = base + tid;
        float sc = -INFINITY;
        if (j <= pos) {
            const int page = table[j / P];
            const T* pg = pages + (int64_t)page * page_stride;
            const int64_t c_at = (int64_t)(j % P) * rank;
            const T* c = pg + c_at;
            const T* kr = pg + (int64_t)2 * P * rank + (int64_t)(j % P) * rot;
            float dot = 0.f;
            for (int i = 0; i < rank; ++i) dot += qa[i] * to_f32<T>(c[i]);
            for (int i = 0; i < rot; ++i) dot += qr[i] * to_f32<T>(kr[i]);
            sc = dot * scale;
            where[tid] = (int64_t)page * page_stride + c_at;
        }
        const float m_new = fmaxf(m, block_max(sc, red));
        const float p = j <= pos ? expf(sc - m_new) : 0.f;
        pw[tid] = p;
        const float tile_sum = block_sum(p, red);  // (its barriers also publish pw and where)
        const float alpha = expf(m - m_new);
        l = l * alpha + tile_sum;
        m = m_new;
        const int count = min(LAT_TILE, pos - base + 1);
#pragma unroll
        for (int k = 0; k < LAT_MAX_RANK_PER_THREAD; ++k) {
            const int r = tid + k * LAT_TILE;
            if (r < rank) {
                float a = acc[k] * alpha;
                for (int jj = 0; jj < count; ++jj) a += pw[jj] * to_f32<T>(pages[where[jj] + r]);
                acc[k] = a;
            }
        }
        __syncthreads();  // pw and where are rewritten by the next tile
    }
    T* o = out + ((int64_t)n * H + h) * rank;
#pragma unroll
    for (int k = 0; k < LAT_MAX_RANK_PER_THREAD; ++k) {
        const int r = tid + k * LAT_TILE;
        if (r < rank) o[r] = from_f32<T>(acc[k] / l);
    }
}

extern "C" int lle_latent_attention_generic(const void* q_lat, int q_lat_dtype, int64_t ql_stride_n,
                                            int64_t ql_stride_h, const void* q_rot, const void* pages,
                                            int64_t page_stride, int P, int rank, int rot, const void* block_table,
                                            int max_pages, const void* seq_slots, const void* cu_tokens,
                                            const void* kv_lens, const void* token_seq, const void* sink, int window,
                                            float scale, void* out, int N, int H, int dtype, hipStream_t stream) {
    if (N <= 0 || H <= 0) return 0;
    if (rank <= 0 || rank > LAT_TILE * LAT_MAX_RANK_PER_THREAD || rot < 0 || P <= 0 || H > 65535)
        return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32 && q_lat_dtype != LLE_F32) return (int)hipErrorInvalidValue;
    const dim3 grid(N, H);
    const size_t lds = (size_t)(rank + rot + LAT_TILE + 16) * sizeof(float) + LAT_TILE * sizeof(int64_t);
#define LAT_ARGS(T, TQ)                                                                                          \
    (const TQ*)q_lat, ql_stride_n, ql_stride_h, (const float*)q_rot, (const T*)pages, page_stride, P, rank, rot, \
        (const int32_t*)block_table, max_pages, (const int32_t*)seq_slots, (const int32_t*)cu_tokens,            \
        (const int32_t*)kv_lens, (const int32_t*)token_seq, (const float*)sink, window, scale, (T*)out, H
    if (dtype == LLE_F32)
        latent_attention_generic_kernel<float, float><<<grid, LAT_TILE, lds, stream>>>(LAT_ARGS(float, float));
    else if (q_lat_dtype == LLE_F32)
        latent_attention_generic_kernel<bf16_t, float><<<grid, LAT_TILE, lds, stream>>>(LAT_ARGS(bf16_t, float));
    else
        latent_attention_generic_kernel<bf16_t, bf16_t><<<grid, LAT_TILE, lds, stream>>>(LAT_ARGS(bf16_t, bf16_t));
#undef LAT_ARGS
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// bfloat16 on the matrix cores.  The rows of a request are its (token, head) pairs, token after
// token; a workgroup of four wavefronts takes one tile of 16 rows over a range of 64-key steps:
//   S^T = K Q^T      A = [16 keys x 32 elements] of [c | k_rot], B = the queries (in LDS):
//                    wavefront w takes the keys 16 w .. 16 w + 15 of the step
//   O^T += C^T P^T   A = [16 latent elements x 32 keys] of the transposed latents, B = P^T:
//                    wavefront w takes a quarter of the latent's elements over all 64 keys
// With v_mfma_f32_16x16x32_bf16 lane (c = lane / 16, r = lane % 16) holds of a result tile column r,
// rows 4c .. 4c + 3: four keys of query row r after the first product.  The rows' maxima and the
// weights P (bfloat16, [row][key]) cross between the wavefronts through LDS, two barriers a step;
// the buffers take turns, so a step's writes never meet the reads of the step before.  All of a
// step's operands (one K tile and the wavefront's share of the transposed latents) are asked for
// at the top of the step, straight from the pages, and travel together.  The quarter of the
// accumulators per wavefront is what leaves registers for that.  With `nsplit` > 1 a tile's keys
// are cut into ranges whose unnormalised results (and m, l) go to a workspace and are merged by
// latent_combine_kernel; the sink (m = sink, l = 1) belongs to the first range.
// RT = row tiles of one workgroup (1 or 2): with two, the step's operands serve 32 rows.
// RK = 32-element steps over the latent (rank <= 32 RK, padded with zeros), RR the same for k_rot.
// PAD: rank < 32 RK or rot < 32 RR, and the operands' tails are filled with zeros under a condition.
// Without it every load is unconditional (a key outside the tile's range is read from the nearest one
// inside it and masked afterwards; the pages hold finite numbers everywhere).
// ---------------------------------------------------------------------------------------------
typedef bf16_t lbf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t lbf16x4 __attribute__((ext_vector_type(4)));
typedef float lf32x4 __attribute__((ext_vector_type(4)));
#define LAT_NEG_BIG (-1.0e30f)
#define LAT_LOG2E 1.4426950408889634f
#define LAT_STEP 64
#define LAT_P_STRIDE 72  // bfloat16 elements between the rows of P in LDS: 64 keys and 16 bytes to spread the banks

__device__ __forceinline__ lbf16x8 lat_zero8() {
    lbf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16_t)0.0f;
    return z;
}

template <int RK, int RR, bool PAD, int RT>
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ q_lat, int64_t ql_stride_n, int64_t ql_stride_h, const float* __restrict__ q_rot,
    const bf16_t* __restrict__ pages, int64_t page_stride, int P, int rank, int rot,
    const int32_t* __restrict__ block_table, int max_pages, const int32_t* __restrict__ seq_slots,
    const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ kv_lens, const float* __restrict__ sink,
    int window, float scale, bf16_t* __restrict__ out, float* __restrict__ ws_o, float* __restrict__ ws_ml, int H,
    int tiles_max, int nsplit) {
    constexpr int NT = RK / 2;  // value tiles (16 latent elements each) of one wavefront, of 2 RK
    __shared__ float s_max[2][RT][4][16];
    __shared__ __attribute__((aligned(16))) bf16_t s_p[2][RT][16][LAT_P_STRIDE];
    __shared__ float s_l[RT][4][16];
    __shared__ __attribute__((aligned(16))) bf16_t s_q[RT][16][32 * (RK + RR) + 8];  // (8 more: rows 16 bytes off the banks)
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE, c = lane / 16, r = lane % 16;
    int item = blockIdx.x;
    const int split = item % nsplit;
    item /= nsplit;
    // the last tiles of a request see the most keys: they start first, so that no long tile is left for the end
    const int tile = tiles_max - 1 - item % tiles_max, s = item / tiles_max;
    const int q0 = cu_tokens[s], q_len = cu_tokens[s + 1] - q0;
    const int rows = q_len * H;
    const int row0 = tile * 16 * RT;  // the workgroup's RT tiles of 16 rows: row0 .. row0 + 16 RT - 1
    if (row0 >= rows) return;  // (the whole workgroup)
    const int past = kv_lens[s] - q_len;
    bool valid[RT];
    int tok[RT], head[RT], pos[RT], lo[RT];
#pragma unroll
    for (int u = 0; u < RT; ++u) {
        const int rho = row0 + 16 * u + r;
        valid[u] = rho < rows;
        tok[u] = valid[u] ? rho / H : 0;
        head[u] = valid[u] ? rho % H : 0;
        pos[u] = valid[u] ? past + tok[u] : -1;  // a row that does not exist sees nothing
        lo[u] = window > 0 ? max(0, pos[u] - window + 1) : 0;
    }
    const int t_first = row0 / H, t_last = min(q_len - 1, (row0 + 16 * RT - 1) / H);
    const int kmax = past + t_last;  // the workgroup's keys: lo_min .. kmax
    const int lo_min = window > 0 ? max(0, past + t_first - window + 1) : 0;
    const int32_t* table = block_table + (int64_t)seq_slots[s] * max_pages;

    // the tiles' queries wait in LDS as the B operands of the first product: row r, elements 32 i + 8 c .. + 7
    // for lane (c, r) and step i; every wavefront writes a quarter of the steps and reads them all
#pragma unroll
    for (int u = 0; u < RT; ++u) {
        const bf16_t* ql = q_lat + (int64_t)(q0 + tok[u]) * ql_stride_n + (int64_t)head[u] * ql_stride_h;
        const float* qr = q_rot + ((int64_t)(q0 + tok[u]) * H + head[u]) * rot;
        for (int i = wave; i < RK + RR; i += 4) {
            lbf16x8 v = lat_zero8();
            if (i < RK) {
                const int e0 = 32 * i + 8 * c;
                if (valid[u] && e0 < rank) v = *(const lbf16x8*)(ql + e0);
            } else {
                const int e0 = 32 * (i - RK) + 8 * c;
                if (valid[u] && e0 < rot) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = (bf16_t)qr[e0 + e];
                }
            }
            *(lbf16x8*)&s_q[u][r][32 * i + 8 * c] = v;
        }
    }
    __syncthreads();
    lf32x4 o[RT][NT];
    float m[RT], l[RT];
#pragma unroll
    for (int u = 0; u < RT; ++u) {
#pragma unroll
        for (int i = 0; i < NT; ++i) o[u][i] = lf32x4{0.f, 0.f, 0.f, 0.f};
        const bool first = split == 0 && valid[u] && sink != nullptr;
        m[u] = first ? sink[head[u]] * LAT_LOG2E : LAT_NEG_BIG;     // base 2; the same in the row's lanes of every wavefront
        l[u] = (first && c == 0 && wave == 0) ? 1.0f : 0.0f;        // this lane's share of the row's sum
    }
    const float sc2 = scale * LAT_LOG2E;

    const int s_begin = lo_min / LAT_STEP, s_end = kmax / LAT_STEP + 1;
    const int per = (s_end - s_begin + nsplit - 1) / nsplit;
    const int st_lo = s_begin + split * per, st_hi = min(s_end, st_lo + per);
    int buf = 0;
    for (int st = st_lo; st < st_hi; ++st, buf ^= 1) {
        const int j0 = st * LAT_STEP;
        // every operand of the step is asked for here, once for all the workgroup's row tiles
        lbf16x8 ka[RK + RR];
        {
            const int key = min(max(j0 + 16 * wave + r, lo_min), kmax);  // (outside: masked below)
            const bf16_t* pg = pages + (int64_t)table[key / P] * page_stride;
            const bf16_t* kp = pg + (int64_t)(key % P) * rank + 8 * c;
            const bf16_t* krp = pg + (int64_t)2 * P * rank + (int64_t)(key % P) * rot + 8 * c;
#pragma unroll
            for (int ks = 0; ks < RK; ++ks)
                ka[ks] = (!PAD || 32 * ks + 8 * c < rank) ? *(const lbf16x8*)(kp + 32 * ks) : lat_zero8();
#pragma unroll
            for (int kr = 0; kr < RR; ++kr)
                ka[RK + kr] = (!PAD || 32 * kr + 8 * c < rot) ? *(const lbf16x8*)(krp + 32 * kr) : lat_zero8();
        }
        lbf16x8 va[2][NT];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            // this lane's eight keys, inside one page; a group outside the tile's range has no weight and is
            // read from the nearest group inside it
            const int gkey = min(max(j0 + 32 * kk + 8 * c, lo_min & ~7), kmax & ~7);
            const bf16_t* vt = pages + (int64_t)table[gkey / P] * page_stride + (int64_t)P * rank + gkey % P;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                const int n = wave * NT + i;
                va[kk][i] = (!PAD || 16 * n < rank) ? *(const lbf16x8*)(vt + (int64_t)(16 * n + r) * P) : lat_zero8();
            }
        }
        float sv[RT][4];
#pragma unroll
        for (int u = 0; u < RT; ++u) {
            lf32x4 sacc = lf32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < RK + RR; ++i)
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[i], *(const lbf16x8*)&s_q[u][r][32 * i + 8 * c], sacc, 0,
                                                               0, 0);
            float mx = LAT_NEG_BIG;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = j0 + 16 * wave + 4 * c + i;
                sv[u][i] = (key >= lo[u] && key <= pos[u]) ? sacc[i] * sc2 : LAT_NEG_BIG;
                mx = fmaxf(mx, sv[u][i]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, LLE_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, LLE_WAVE));
            if (c == 0) s_max[buf][u][wave][r] = mx;
        }
        __syncthreads();
        float alpha[RT];
#pragma unroll
        for (int u = 0; u < RT; ++u) {
            const float mx = fmaxf(fmaxf(s_max[buf][u][0][r], s_max[buf][u][1][r]),
                                   fmaxf(s_max[buf][u][2][r], s_max[buf][u][3][r]));
            const float m_new = fmaxf(m[u], mx);
            alpha[u] = exp2f(m[u] - m_new);
            lbf16x4 pw;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = sv[u][i] <= 0.5f * LAT_NEG_BIG ? 0.f : exp2f(sv[u][i] - m_new);
                psum += p;
                pw[i] = (bf16_t)p;
            }
            l[u] = l[u] * alpha[u] + psum;
            m[u] = m_new;
            *(lbf16x4*)&s_p[buf][u][r][16 * wave + 4 * c] = pw;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < RT; ++u) {
            if (__any(alpha[u] != 1.0f)) {
#pragma unroll
                for (int i = 0; i < NT; ++i) o[u][i] *= alpha[u];
            }
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const lbf16x8 pb = *(const lbf16x8*)&s_p[buf][u][r][32 * kk + 8 * c];
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    if (!PAD || 16 * (wave * NT + i) < rank)
                        o[u][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[kk][i], pb, o[u][i], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < RT; ++u) {
        l[u] += __shfl_xor(l[u], 16, LLE_WAVE);
        l[u] += __shfl_xor(l[u], 32, LLE_WAVE);
        if (c == 0) s_l[u][wave][r] = l[u];
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < RT; ++u) {
        if (!valid[u]) continue;
        const float lsum = (s_l[u][0][r] + s_l[u][1][r]) + (s_l[u][2][r] + s_l[u][3][r]);
        const int64_t grow = (int64_t)(q0 + tok[u]) * H + head[u];
        if (nsplit == 1) {
            const float inv = 1.0f / lsum;
            bf16_t* orow = out + grow * rank;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                const int n = wave * NT + i;
                if (16 * n < rank) {
                    lbf16x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (bf16_t)(o[u][i][e] * inv);
                    *(lbf16x4*)(orow + 16 * n + 4 * c) = v;
                }
            }
        } else {
            float* wo = ws_o + (grow * nsplit + split) * rank;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                const int n = wave * NT + i;
                if (16 * n < rank) *(lf32x4*)(wo + 16 * n + 4 * c) = o[u][i];
            }
            if (c == 0 && wave == 0) {
                ws_ml[(grow * nsplit + split) * 2] = m[u];
                ws_ml[(grow * nsplit + split) * 2 + 1] = lsum;
            }
        }
    }
}

// grid (rows, ceil(rank / 256)): the ranges' results weighted by 2^(m_i - max m) and normalised, one element a thread
__global__ __launch_bounds__(256) void latent_combine_kernel(const float* __restrict__ ws_o,
                                                              const float* __restrict__ ws_ml,
                                                              bf16_t* __restrict__ out, int rank, int nsplit) {
    __shared__ float weight[64];
    const int64_t row = blockIdx.x;
    const float* ml = ws_ml + row * nsplit * 2;
    float M = LAT_NEG_BIG;
    for (int i = 0; i < nsplit; ++i) M = fmaxf(M, ml[2 * i]);
    float L = 0.f;
    for (int i = 0; i < nsplit; ++i) L += ml[2 * i + 1] * exp2f(ml[2 * i] - M);
    if (threadIdx.x < nsplit) weight[threadIdx.x] = exp2f(ml[2 * threadIdx.x] - M) / L;
    __syncthreads();
    const int e = blockIdx.y * blockDim.x + threadIdx.x;
    if (e >= rank) return;
    const float* src = ws_o + row * nsplit * rank + e;
    float acc = 0.f;
#pragma unroll 8
    for (int i = 0; i < nsplit; ++i) acc += src[(int64_t)i * rank] * weight[i];
    out[row * rank + e] = (bf16_t)acc;
}

// q_lat bfloat16 [N, H, rank] with strides that are multiples of 8; rank a multiple of 16 up to 512, rot a
// multiple of 8 up to 64, P a multiple of 16.  `tiles_max` = ceil(max_q_len * H / (16 row_tiles)).  nsplit > 1 needs
// ws_o float32 [N H nsplit rank] and ws_ml float32 [N H nsplit 2].
extern "C" int lle_latent_attention_mfma(const void* q_lat, int64_t ql_stride_n, int64_t ql_stride_h,
                                         const void* q_rot, const void* pages, int64_t page_stride, int P, int rank,
                                         int rot, const void* block_table, int max_pages, const void* seq_slots,
                                         const void* cu_tokens, const void* kv_lens, const void* sink, int window,
                                         float scale, void* out, void* ws_o, void* ws_ml, int N, int S, int H,
                                         int tiles_max, int nsplit, int row_tiles, hipStream_t stream) {
    if (N <= 0 || S <= 0 || H <= 0 || tiles_max <= 0) return 0;
    if (rank <= 0 || rank > 512 || rank % 16 || rot < 0 || rot > 64 || rot % 8 || P <= 0 || P % 16 ||
        ql_stride_n % 8 || ql_stride_h % 8 || page_stride % 8 || nsplit < 1 || nsplit > 64 ||
        (nsplit > 1 && (!ws_o || !ws_ml)))
        return (int)hipErrorInvalidValue;
    const int64_t items = (int64_t)S * tiles_max * nsplit;
    if (items > 0x7fffffff) return (int)hipErrorInvalidValue;
    const int RK = rank <= 64 ? 2 : rank <= 128 ? 4 : rank <= 256 ? 8 : 16;
    const int RR = rot <= 32 ? 1 : 2;
    const bool pad = rank != 32 * RK || rot != 32 * RR;
    if (row_tiles != 1 && row_tiles != 2) return (int)hipErrorInvalidValue;
#define LAT_LAUNCH(K, R)                                                                                              \
    if (pad && row_tiles == 1)                                                                                        \
        LAT_LAUNCH_(K, R, true, 1);                                                                                   \
    else if (pad)                                                                                                     \
        LAT_LAUNCH_(K, R, true, 2);                                                                                   \
    else if (row_tiles == 1)                                                                                          \
        LAT_LAUNCH_(K, R, false, 1);                                                                                  \
    else                                                                                                              \
        LAT_LAUNCH_(K, R, false, 2)
#define LAT_LAUNCH_(K, R, PADDED, TILES)                                                                              \
    latent_attention_mfma_kernel<K, R, PADDED, TILES><<<(int)items, 256, 0, stream>>>(                                \
        (const bf16_t*)q_lat, ql_stride_n, ql_stride_h, (const float*)q_rot, (const bf16_t*)pages, page_stride, P,    \
        rank, rot, (const int32_t*)block_table, max_pages, (const int32_t*)seq_slots, (const int32_t*)cu_tokens,      \
        (const int32_t*)kv_lens, (const float*)sink, window, scale, (bf16_t*)out, (float*)ws_o, (float*)ws_ml, H,     \
        tiles_max, nsplit)
    if (RR == 1) {
        if (RK == 2) { LAT_LAUNCH(2, 1); }
        else if (RK == 4) { LAT_LAUNCH(4, 1); }
        else if (RK == 8) { LAT_LAUNCH(8, 1); }
        else { LAT_LAUNCH(16, 1); }
    } else {
        if (RK == 2) { LAT_LAUNCH(2, 2); }
        else if (RK == 4) { LAT_LAUNCH(4, 2); }
        else if (RK == 8) { LAT_LAUNCH(8, 2); }
        else { LAT_LAUNCH(16, 2); }
    }
#undef LAT_LAUNCH
#undef LAT_LAUNCH_
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (nsplit > 1) latent_combine_kernel<<<dim3(N * H, (rank + 255) / 256), 256, 0, stream>>>((const float*)ws_o, (const float*)ws_ml, (bf16_t*)out, rank, nsplit);
    LLE_RETURN_LAUNCH_STATUS();
}
