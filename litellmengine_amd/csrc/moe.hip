// Mixture of experts: the router's choice and the chosen experts' gated feed-forwards, with the
// experts indexed on the device (nothing about the choice travels to the host).
//
//   ids, gains = top-k of (logits + bias), gains = softmax over the chosen logits     moe_route
//   act[p]   = silu(Wg[e_p] x_n) * (Wu[e_p] x_n)      p = (token n, k-th choice)      moe_gate_up
//   out[n]   = sum_k gains[n, k] * Wd[e_(n,k)] act[(n, k)]        32-bit              moe_down
//
// Few tokens (decoding): every (token, choice) pair streams the rows of its expert's weights, a
// wavefront per output element.  Many tokens (prompt portions): the pairs are first put in the order of
// their experts (a counting sort on the device), then tiles of 16 pairs of one expert go through the
// matrix cores against that expert's weights (moe_*_tile kernels, bfloat16), so that an expert's
// weights are read once per tile and not once per token.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define MOE_MAX_TOP 16

// one thread per token: the `top` largest of logits + bias (the lower index wins a tie), then
// the softmax over those alone.  ids int32 [N, top], gains float32 [N, top].
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits,
                                                         const float* __restrict__ bias, int32_t* __restrict__ ids,
                                                         float* __restrict__ gains, int N, int E, int top) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const float* row = logits + (int64_t)n * E;
    int chosen[MOE_MAX_TOP];
    float value[MOE_MAX_TOP];
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
            if (taken) continue;
            const float v = row[e] + bias[e];
            if (best < 0 || v > bv) {
                best = e;
                bv = v;
            }
        }
        chosen[k] = best;
        value[k] = bv;
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
                             hipStream_t stream) {
    if (N <= 0) return 0;
    if (top <= 0 || top > MOE_MAX_TOP || top > E) return (int)hipErrorInvalidValue;
    moe_route_kernel<<<(N + 255) / 256, 256, 0, stream>>>((const float*)logits, (const float*)bias, (int32_t*)ids,
                                                           (float*)gains, N, E, top);
    LLE_RETURN_LAUNCH_STATUS();
}

template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ a, const T* __restrict__ b, int K) {
    float acc = 0.f;
    for (int k = threadIdx.x % LLE_WAVE; k < K; k += LLE_WAVE) acc += to_f32<T>(a[k]) * to_f32<T>(b[k]);
    return wave_sum(acc);
}

// grid (pairs, ceil(F / 4)), 4 wavefronts: wavefront w makes act[p, f], f = 4 blockIdx.y + w
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const int32_t* __restrict__ ids,
                                                           const T* __restrict__ gate_up, T* __restrict__ act, int top,
                                                           int F, int K) {
    const int p = blockIdx.x;
    const int f = blockIdx.y * 4 + threadIdx.x / LLE_WAVE;
    if (f >= F) return;
    const int e = ids[p];
    const T* xr = x + (int64_t)(p / top) * K;
    const T* w = gate_up + (int64_t)e * 2 * F * K;
    const float g = wave_dot<T>(xr, w + (int64_t)f * K, K);
    const float u = wave_dot<T>(xr, w + (int64_t)(F + f) * K, K);
    if (threadIdx.x % LLE_WAVE == 0) act[(int64_t)p * F + f] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

// grid (tokens, ceil(H / 4)), 4 wavefronts: wavefront w makes out[n, o], o = 4 blockIdx.y + w
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const int32_t* __restrict__ ids,
                                                        const float* __restrict__ gains, const T* __restrict__ down,
                                                        float* __restrict__ out, int top, int F, int H) {
    const int n = blockIdx.x;
    const int o = blockIdx.y * 4 + threadIdx.x / LLE_WAVE;
    if (o >= H) return;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        const int p = n * top + k;
        const T* w = down + ((int64_t)ids[p] * H + o) * F;
        total += gains[p] * wave_dot<T>(act + (int64_t)p * F, w, F);
    }
    if (threadIdx.x % LLE_WAVE == 0) out[(int64_t)n * H + o] = total;
}

// x [N, K], ids/gains [N, top], gate_up [E, 2 F, K], down [E, H, F], act [N top, F] (scratch), out float32 [N, H]
extern "C" int lle_moe_experts(const void* x, const void* ids, const void* gains, const void* gate_up,
                               const void* down, void* act, void* out, int N, int top, int F, int K, int H, int dtype,
                               hipStream_t stream) {
    if (N <= 0) return 0;
    if (top <= 0 || (int64_t)N * top > 0x7fffffff) return (int)hipErrorInvalidValue;
    const dim3 g1(N * top, (F + 3) / 4), g2(N, (H + 3) / 4);
    if (g1.y > 65535 || g2.y > 65535) return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32) {
        moe_gate_up_kernel<float><<<g1, 256, 0, stream>>>((const float*)x, (const int32_t*)ids, (const float*)gate_up,
                                                           (float*)act, top, F, K);
        moe_down_kernel<float><<<g2, 256, 0, stream>>>((const float*)act, (const int32_t*)ids, (const float*)gains,
                                                        (const float*)down, (float*)out, top, F, H);
    } else {
        moe_gate_up_kernel<bf16_t><<<g1, 256, 0, stream>>>((const bf16_t*)x, (const int32_t*)ids,
                                                            (const bf16_t*)gate_up, (bf16_t*)act, top, F, K);
        moe_down_kernel<bf16_t><<<g2, 256, 0, stream>>>((const bf16_t*)act, (const int32_t*)ids, (const float*)gains,
                                                         (const bf16_t*)down, (float*)out, top, F, H);
    }
    LLE_RETURN_LAUNCH_STATUS();
}
