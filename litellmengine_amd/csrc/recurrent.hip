// Gated recurrences over the tokens of a step.
//
// minGRU:  z = sigmoid(a + bz), c = g(u + bx) with g(u) = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
//          S <- (1 - z) S + z c   element by element, y = S * silu(gate).
// `zxg` holds a, u and gate of every token side by side ([N, 3 W], float32 or bfloat16); the
// biases are float32; the state is float32 [slots + 1, W], one row per request slot, read at
// the start of a request's tokens and written back after the last.  All arithmetic is 32-bit.
//
// The recurrence is linear in S: S_out = A S_in + B with A = prod (1 - z), so the tokens of a
// long portion are cut into pieces that are scanned side by side:
//   a short portion (or a decoded token): one thread per (request, channel) walks the tokens;
//   a long portion: every piece first reduces its (A, B); a short walk over the pieces' (A, B) gives the
//   state each piece starts from (and the request's new state); then every piece walks its tokens.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

struct GruStep {
    float z, c;
};

__device__ __forceinline__ GruStep gru_gates(const void* zxg, int dtype, int64_t row, int W, int ch, float bz,
                                             float bx) {
    const float a = load_as_f32(zxg, row * 3 * W + ch, dtype) + bz;
    const float u = load_as_f32(zxg, row * 3 * W + W + ch, dtype) + bx;
    GruStep g;
    g.z = sigmoid_f(a);
    g.c = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    return g;
}

// grid (requests, pieces, channel blocks).  pieces == 1: the whole walk (`pass` 1).  pieces > 1: `pass` 0
// leaves (A, B) of every piece in part[(s * pieces + piece) * 3 W ...]; mingru_carry_kernel turns them
// into the state each piece starts from (and writes the request's new state); `pass` 1 walks the tokens.
template <typename TO>
__global__ __launch_bounds__(256) void mingru_scan_kernel(const void* __restrict__ zxg, int in_dtype,
                                                           const float* __restrict__ z_bias,
                                                           const float* __restrict__ x_bias,
                                                           float* __restrict__ state,
                                                           const int32_t* __restrict__ seq_slots,
                                                           const int32_t* __restrict__ cu_tokens,
                                                           TO* __restrict__ out, float* __restrict__ part, int W,
                                                           int pieces, int pass) {
    const int s = blockIdx.x, piece = blockIdx.y;
    const int ch = blockIdx.z * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    const int q0 = cu_tokens[s], q1 = cu_tokens[s + 1];
    const int len = q1 - q0;
    const int per = (len + pieces - 1) / pieces;
    const int t0 = q0 + piece * per;
    const int t1 = min(q1, t0 + per);
    const float bz = z_bias[ch], bx = x_bias[ch];
    float* p = part + ((int64_t)s * pieces + piece) * 3 * W;
    if (pieces > 1 && pass == 0) {
        float A = 1.f, B = 0.f;
#pragma unroll 4
        for (int t = t0; t < t1; ++t) {
            const GruStep g = gru_gates(zxg, in_dtype, t, W, ch, bz, bx);
            A *= 1.f - g.z;
            B = (1.f - g.z) * B + g.z * g.c;
        }
        p[ch] = A;
        p[W + ch] = B;
        return;
    }
    float* st = state + (int64_t)seq_slots[s] * W + ch;
    float S = pieces > 1 ? p[2 * W + ch] : *st;  // (pieces > 1: the carry that mingru_carry_kernel left)
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        const GruStep g = gru_gates(zxg, in_dtype, t, W, ch, bz, bx);
        S = (1.f - g.z) * S + g.z * g.c;
        const float gate = load_as_f32(zxg, (int64_t)t * 3 * W + 2 * W + ch, in_dtype);
        out[(int64_t)t * W + ch] = from_f32<TO>(S * (gate * sigmoid_f(gate)));
    }
    if (pieces == 1) *st = S;
}

// one thread per (request, channel): walks the pieces' (A, B) in order, leaves beside them the state each
// piece starts from, and writes the state after the last piece back to the request's row.  (A, B) are read
// eight pieces at a time, so that their loads travel together: nothing written here is read here.
__global__ __launch_bounds__(64) void mingru_carry_kernel(float* __restrict__ state,
                                                           const int32_t* __restrict__ seq_slots,
                                                           float* __restrict__ part, int W, int pieces) {
    const int s = blockIdx.x;
    const int ch = blockIdx.y * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    float* st = state + (int64_t)seq_slots[s] * W + ch;
    float* base = part + (int64_t)s * pieces * 3 * W + ch;
    float S = *st;
    for (int k0 = 0; k0 < pieces; k0 += 8) {
        float A[8], B[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = min(k0 + i, pieces - 1);
            A[i] = __builtin_nontemporal_load(base + (int64_t)k * 3 * W);
            B[i] = __builtin_nontemporal_load(base + (int64_t)k * 3 * W + W);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (k0 + i < pieces) {
                base[(int64_t)(k0 + i) * 3 * W + 2 * W] = S;
                S = A[i] * S + B[i];
            }
        }
    }
    *st = S;
}

// `part`: float32 [S * pieces * 3 W] when pieces > 1 (else unused): A, B and the starting state of every piece
extern "C" int lle_mingru_scan(const void* zxg, int in_dtype, const void* z_bias, const void* x_bias, void* state,
                               const void* seq_slots, const void* cu_tokens, void* out, int out_dtype, void* part,
                               int S, int W, int pieces, hipStream_t stream) {
    if (S <= 0 || W <= 0) return 0;
    if (pieces < 1 || (pieces > 1 && part == nullptr) || pieces > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid(S, pieces, (W + 255) / 256);
    for (int pass = (pieces > 1 ? 0 : 1); pass < 2; ++pass) {
        if (out_dtype == LLE_F32)
            mingru_scan_kernel<float><<<grid, 256, 0, stream>>>(zxg, in_dtype, (const float*)z_bias,
                                                                 (const float*)x_bias, (float*)state,
                                                                 (const int32_t*)seq_slots, (const int32_t*)cu_tokens,
                                                                 (float*)out, (float*)part, W, pieces, pass);
        else
            mingru_scan_kernel<bf16_t><<<grid, 256, 0, stream>>>(zxg, in_dtype, (const float*)z_bias,
                                                                  (const float*)x_bias, (float*)state,
                                                                  (const int32_t*)seq_slots,
                                                                  (const int32_t*)cu_tokens, (bf16_t*)out,
                                                                  (float*)part, W, pieces, pass);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
        if (pass == 0) {
            mingru_carry_kernel<<<dim3(S, (W + 63) / 64), 64, 0, stream>>>((float*)state, (const int32_t*)seq_slots,
                                                                                (float*)part, W, pieces);
            e = hipGetLastError();
            if (e != hipSuccess) return (int)e;
        }
    }
    return 0;
}
