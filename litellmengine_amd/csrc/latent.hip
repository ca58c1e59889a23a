// Latent attention: the cache holds, per token, one latent row c [rank] and one rotated key part
// k_rot [rot] shared by all heads; a page is [page_size][rank] of c followed by
// [page_size][rot] of k_rot.  Queries arrive already carried into the latent space
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
    T* kr = page + (int64_t)P * rank + (int64_t)(slot % P) * rot;
    for (int i = threadIdx.x; i < rank; i += blockDim.x)
        c[i] = from_f32<T>(to_f32<T>(row[i]) * inv * load_as_f32(norm_w, i, w_dtype));
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

    float m = sink[h], l = 1.0f;  // the sink: a key with score `sink` and no value
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
            const T* kr = pg + (int64_t)P * rank + (int64_t)(j % P) * rot;
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
