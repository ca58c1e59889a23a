// A recurrence with a matrix state per head and a decay made from the data (the "wkv" mixer):
//
//   mix_s[t] = h[t] + (h[t-1] - h[t]) * mu_s         s of several; h[-1] is the state's saved row     shift_mix
//   decay    = exp(-exp(x + w0))                      per head and key channel, 32-bit
//   o_t[j]   = sum_i r_t[i] (S[i][j] + u[i] k_t[i] v_t[j])                                            wkv_scan
//   S[i][j] <- decay_t[i] S[i][j] + k_t[i] v_t[j]
//   y_t      = o_t / rms(o_t) * norm_w * silu(g_t)    per head, eps inside the root
//
// The state is float32 [head][key i][value j] per request slot, followed in the same row by the last
// token's mixer input h (what the next step's first token is shifted against).  A thread owns one
// value channel j of one head and keeps S[:, j] in registers; r, k and the decays of a few tokens
// are staged in LDS, where every thread reads the same word at a time (a broadcast).
//
// The state is linear in what came before: S_out = diag(A) S_in + B, A the product of a stretch's
// decays.  A long portion is therefore cut into pieces that are walked side by side:
//   pass 1  every piece but a request's last, from a zero state: A and B                (no outputs)
//   carry   a short walk over the pieces leaves every piece's entry state
//   pass 2  every piece again from its entry state, with outputs; the last writes the state back
// A step of single tokens, or of short portions, is one launch from the state itself.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define WKV_TC 8  // tokens staged at a time

// out[m][n][:] = x[n] + (prev - x[n]) * mu[m], prev = x[n - 1], or the saved row of the request's state
// for the first token of its portion.  grid = tokens.
template <typename T>
__global__ __launch_bounds__(256) void shift_mix_kernel(const T* __restrict__ x, const float* __restrict__ state,
                                                         int64_t state_stride, int prev_offset,
                                                         const float* __restrict__ mu, const int32_t* __restrict__ token_seq,
                                                         const int32_t* __restrict__ cu_tokens,
                                                         const int32_t* __restrict__ seq_slots, T* __restrict__ out, int N,
                                                         int W, int M) {
    const int64_t n = blockIdx.x;
    const int s = token_seq[n];
    const bool first = cu_tokens[s] == n;
    const float* saved = state + (int64_t)seq_slots[s] * state_stride + prev_offset;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        const float h = to_f32<T>(x[n * W + e]);
        const float p = first ? saved[e] : to_f32<T>(x[(n - 1) * W + e]);
        for (int m = 0; m < M; ++m)
            out[((int64_t)m * N + n) * W + e] = from_f32<T>(h + (p - h) * mu[(int64_t)m * W + e]);
    }
}

extern "C" int lle_shift_mix(const void* x, const void* state, int64_t state_stride, int prev_offset, const void* mu,
                             const void* token_seq, const void* cu_tokens, const void* seq_slots, void* out, int N, int W,
                             int M, int dtype, hipStream_t stream) {
    if (N <= 0 || W <= 0 || M <= 0) return 0;
    if (dtype == LLE_F32)
        shift_mix_kernel<float><<<N, 256, 0, stream>>>((const float*)x, (const float*)state, state_stride, prev_offset,
                                                        (const float*)mu, (const int32_t*)token_seq,
                                                        (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (float*)out,
                                                        N, W, M);
    else
        shift_mix_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)x, (const float*)state, state_stride, prev_offset,
                                                         (const float*)mu, (const int32_t*)token_seq,
                                                         (const int32_t*)cu_tokens, (const int32_t*)seq_slots, (bf16_t*)out,
                                                         N, W, M);
    LLE_RETURN_LAUNCH_STATUS();
}

struct WkvArgs {
    const float* r;      // [N, H dim]
    const float* k;
    const float* v;
    const float* wraw;   // [N, H dim]: the decay's exponent before w0 is added
    const float* w0;     // [H dim]
    const float* u;      // [H dim]
    const void* g;       // [N, H dim], the output gate's input, activation type
    const void* norm_w;  // [H dim]
    int norm_dtype;
    float eps;
    const void* x;       // [N, W]: the mixer's input, whose last row of a request is saved
    float* state;        // [slots, state_stride]
    int64_t state_stride;
    int prev_offset;
    const int32_t* seq_slots;
    const int32_t* cu_tokens;
    void* out;           // [N, H dim], activation type
    int H, dim, W;
    int pieces, piece_len;
    float* part;         // [S, pieces, H, dim * dim + dim]: B (then the entry state) and A of every piece
};

#define WKV_FROM_STATE 0  // one walk over a request's tokens
#define WKV_SUMMARY 1     // pass 1
#define WKV_FROM_ENTRY 2  // pass 2

// grid = (requests x pieces, heads).  KD >= dim (a multiple of 16) key channels are kept; a workgroup is WKV_IG
// groups of JT = 64, 128 or 256 threads: thread (ig, j) owns value channel j and the key channels
// [ig KD / WKV_IG, (ig + 1) KD / WKV_IG) of S[:, j].  The groups' shares of o_t meet in LDS.  (One group that
// walks all key channels is a wavefront that issues one instruction after the other with nobody to fill its
// gaps; four of them on a SIMD do: 251 -> 114 us for 2048 tokens of 32 heads of 64, all three launches.)
// WKV_SUMMARY is pass 1: the same walk from a zero state without outputs, which leaves B and A.
#define WKV_IG 4
template <int KD, typename T, int MODE>
__global__ __launch_bounds__((KD <= 64 ? 64 : KD <= 128 ? 128 : 256) * WKV_IG) void wkv_scan_kernel(WkvArgs a) {
    constexpr bool OUT = MODE != WKV_SUMMARY;
    constexpr int JT = KD <= 64 ? 64 : KD <= 128 ? 128 : 256;
    constexpr int KI = KD / WKV_IG;
    static_assert(KD % WKV_IG == 0, "the key channels are dealt to the groups in equal shares");
    __shared__ float s_r[WKV_TC][KD], s_k[WKV_TC][KD], s_w[WKV_TC][KD], s_u[KD];
    __shared__ float s_o[WKV_IG][WKV_TC][KD];
    __shared__ float s_inv[WKV_TC];
    const int dim = a.dim, HD = a.H * a.dim;
    const int s = blockIdx.x / a.pieces, piece = blockIdx.x % a.pieces;
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    const int j = tid % JT, ig = tid / JT, i0 = ig * KI;
    const int q0 = a.cu_tokens[s], q1 = a.cu_tokens[s + 1];
    const int live = (q1 - q0 + a.piece_len - 1) / a.piece_len;  // pieces of this request that hold tokens
    if (piece >= live) return;
    if (MODE == WKV_SUMMARY && piece == live - 1) return;  // nobody comes after the last piece
    const int t0 = q0 + piece * a.piece_len, t1 = min(q1, t0 + a.piece_len);
    float* st = a.state + (int64_t)a.seq_slots[s] * a.state_stride;
    float* srow = st + (int64_t)h * dim * dim;
    float* prow = a.part ? a.part + ((int64_t)(s * a.pieces + piece) * a.H + h) * (dim * dim + dim) : nullptr;

    float S[KI];
#pragma unroll
    for (int ii = 0; ii < KI; ++ii) {
        const int i = i0 + ii;
        float x = 0.f;
        if (MODE == WKV_FROM_STATE && i < dim && j < dim) x = srow[i * dim + j];
        if (MODE == WKV_FROM_ENTRY && i < dim && j < dim) x = prow[i * dim + j];
        S[ii] = x;
    }
    float A = 1.0f;  // (thread (0, i): the product of the piece's decays of key channel i)
    for (int i = tid; i < KD; i += blockDim.x) s_u[i] = i < dim ? a.u[h * dim + i] : 0.f;

    for (int c0 = t0; c0 < t1; c0 += WKV_TC) {
        const int nt = min(WKV_TC, t1 - c0);
        __syncthreads();  // (the chunk before has been read)
        for (int idx = tid; idx < nt * KD; idx += blockDim.x) {
            const int t = idx / KD, i = idx - t * KD;
            float rr = 0.f, kk = 0.f, ww = 1.0f;
            if (i < dim) {
                const int64_t at = (int64_t)(c0 + t) * HD + h * dim + i;
                rr = a.r[at];
                kk = a.k[at];
                ww = expf(-expf(a.wraw[at] + a.w0[h * dim + i]));
            }
            s_r[t][i] = rr;
            s_k[t][i] = kk;
            s_w[t][i] = ww;
        }
        float vv[WKV_TC];
#pragma unroll
        for (int t = 0; t < WKV_TC; ++t)
            vv[t] = (t < nt && j < dim) ? a.v[(int64_t)(c0 + t) * HD + h * dim + j] : 0.f;
        __syncthreads();
#pragma unroll
        for (int t = 0; t < WKV_TC; ++t) {
            if (t < nt) {
                float o = 0.f;
#pragma unroll
                for (int ii = 0; ii < KI; ++ii) {
                    const int i = i0 + ii;
                    const float kv = s_k[t][i] * vv[t];
                    if (OUT) o = fmaf(s_r[t][i], fmaf(s_u[i], kv, S[ii]), o);
                    S[ii] = fmaf(s_w[t][i], S[ii], kv);
                }
                if (OUT && j < KD) s_o[ig][t][j] = o;
                if (!OUT && ig == 0 && j < dim) A *= s_w[t][j];
            }
        }
        if (OUT) {
            __syncthreads();
            // the groups' shares are added up, and every token's head is divided by its own root mean square:
            // a wavefront per token
            const int wave = tid / LLE_WAVE, lane = tid % LLE_WAVE, waves = blockDim.x / LLE_WAVE;
            for (int t = wave; t < nt; t += waves) {
                float ss = 0.f;
                for (int e = lane; e < dim; e += LLE_WAVE) {
                    float o = s_o[0][t][e];
#pragma unroll
                    for (int g2 = 1; g2 < WKV_IG; ++g2) o += s_o[g2][t][e];
                    s_o[0][t][e] = o;
                    ss += o * o;
                }
                ss = wave_sum(ss);
                if (lane == 0) s_inv[t] = 1.0f / sqrtf(ss / (float)dim + a.eps);
            }
            __syncthreads();
            for (int idx = tid; idx < nt * dim; idx += blockDim.x) {
                const int t = idx / dim, e = idx - t * dim;
                const int64_t at = (int64_t)(c0 + t) * HD + h * dim + e;
                const float gate = to_f32<T>(((const T*)a.g)[at]);
                const float y = s_o[0][t][e] * s_inv[t] * load_as_f32(a.norm_w, h * dim + e, a.norm_dtype) *
                                (gate / (1.0f + expf(-gate)));
                ((T*)a.out)[at] = from_f32<T>(y);
            }
        }
    }
    if (MODE == WKV_SUMMARY) {
        if (j < dim) {
#pragma unroll
            for (int ii = 0; ii < KI; ++ii)
                if (i0 + ii < dim) prow[(i0 + ii) * dim + j] = S[ii];
            if (ig == 0) prow[dim * dim + j] = A;
        }
        return;
    }
    if (piece != live - 1) return;
    if (j < dim) {
#pragma unroll
        for (int ii = 0; ii < KI; ++ii)
            if (i0 + ii < dim) srow[(i0 + ii) * dim + j] = S[ii];
    }
    if (h == 0)  // the request's last input row waits for the next step's first token
        for (int e = tid; e < a.W; e += blockDim.x) st[a.prev_offset + e] = to_f32<T>(((const T*)a.x)[(int64_t)(q1 - 1) * a.W + e]);
}

// grid = (requests, heads, blocks of 256 state elements): a thread walks one element S[i][j] through the
// pieces and leaves every piece's entry state in the place of its B (eight pieces' A and B are asked
// for together: one after the other, each would wait for the memory on its own)
__global__ __launch_bounds__(256) void wkv_carry_kernel(WkvArgs a) {
    const int dim = a.dim;
    const int s = blockIdx.x, h = blockIdx.y;
    const int e = blockIdx.z * blockDim.x + threadIdx.x;
    if (e >= dim * dim) return;
    const int i = e / dim;
    const int q0 = a.cu_tokens[s], q1 = a.cu_tokens[s + 1];
    const int live = (q1 - q0 + a.piece_len - 1) / a.piece_len;
    const int64_t stride = (int64_t)a.H * (dim * dim + dim);
    float* base = a.part + ((int64_t)s * a.pieces * a.H + h) * (dim * dim + dim);
    float S = a.state[(int64_t)a.seq_slots[s] * a.state_stride + (int64_t)h * dim * dim + e];
    for (int p0 = 0; p0 < live; p0 += 8) {
        float A[8], B[8];
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            const int p = min(p0 + n, live - 1);
            B[n] = base[p * stride + e];
            A[n] = base[p * stride + dim * dim + i];
        }
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            if (p0 + n < live) {
                base[(p0 + n) * stride + e] = S;
                S = A[n] * S + B[n];  // (the last piece has left no A and B; what S becomes there is not used)
            }
        }
    }
}

template <int KD, typename T>
static int wkv_launch(const WkvArgs& a, int S, hipStream_t stream) {
    const int threads = (KD <= 64 ? 64 : KD <= 128 ? 128 : 256) * WKV_IG;
    const dim3 grid(S * a.pieces, a.H);
    if (a.pieces == 1) {
        wkv_scan_kernel<KD, T, WKV_FROM_STATE><<<grid, threads, 0, stream>>>(a);
        return (int)hipGetLastError();
    }
    wkv_scan_kernel<KD, T, WKV_SUMMARY><<<grid, threads, 0, stream>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    wkv_carry_kernel<<<dim3(S, a.H, (a.dim * a.dim + 255) / 256), 256, 0, stream>>>(a);
    e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    wkv_scan_kernel<KD, T, WKV_FROM_ENTRY><<<grid, threads, 0, stream>>>(a);
    return (int)hipGetLastError();
}

extern "C" int lle_wkv_max_dim(void) { return 256; }

// r, k, v, wraw float32 [N, H dim]; g, x, out in `dtype`; state float32 rows of `state_stride` floats: H dim dim of
// the matrix state, the saved input row at `prev_offset`.  `pieces` > 1 needs `part`, float32
// [S pieces H (dim dim + dim)]; every request has at most pieces * piece_len tokens.
extern "C" int lle_wkv_scan(const void* r, const void* k, const void* v, const void* wraw, const void* w0, const void* u,
                            const void* g, const void* norm_w, int norm_dtype, float eps, const void* x, void* state,
                            int64_t state_stride, int prev_offset, const void* seq_slots, const void* cu_tokens, void* out,
                            int S, int H, int dim, int W, int pieces, int piece_len, void* part, int dtype,
                            hipStream_t stream) {
    if (S <= 0 || H <= 0) return 0;
    if (dim <= 0 || dim > 256 || pieces < 1 || piece_len < 1 || (pieces > 1 && part == nullptr) || H > 65535 ||
        (int64_t)S * pieces > 0x7fffffff)
        return (int)hipErrorInvalidValue;
    WkvArgs a{(const float*)r, (const float*)k, (const float*)v, (const float*)wraw, (const float*)w0, (const float*)u, g,
              norm_w, norm_dtype, eps, x, (float*)state, state_stride, prev_offset, (const int32_t*)seq_slots,
              (const int32_t*)cu_tokens, out, H, dim, W, pieces, piece_len, (float*)part};
#define WKV_CASE(KD)                                                                    \
    if (dim <= KD)                                                                      \
        return dtype == LLE_F32 ? wkv_launch<KD, float>(a, S, stream) : wkv_launch<KD, bf16_t>(a, S, stream);
    WKV_CASE(16)
    WKV_CASE(32)
    WKV_CASE(48)
    WKV_CASE(64)
    WKV_CASE(96)
    WKV_CASE(128)
    WKV_CASE(192)
    WKV_CASE(256)
#undef WKV_CASE
    return (int)hipErrorInvalidValue;
}
