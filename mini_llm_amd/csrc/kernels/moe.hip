// A mixture of small feed-forward experts, for gfx950: the router and the activation between the experts' two
// products. Router logits, softmax and weights are fp32 whatever the activation dtype.
//
// The experts' first products are one joined product (rows [expert 0 | expert 1 | ... | shared expert]); the
// activation kernel squares the rectified values and multiplies every expert's block by the token's weight for that
// expert (zero for an expert that was not chosen, one for the shared expert), so that the experts' second products are
// one joined product as well: sum_e w_e W_down,e a_e = [W_down,0 | W_down,1 | ...] [w_0 a_0; w_1 a_1; ...].
#include "common.h"

#define MOE_MAX_EXPERTS 256

namespace {

// One wavefront per token: logits z_e = w[e, :] . h (fp32 sums), scores softmax(z) over all experts, the `top`
// largest scores chosen (the lower index wins a tie), weights[t, e] = scale * score_e for them and 0 for the others.
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, int ldh, const float* __restrict__ w, int n_tokens, int D, int E, int top, float scale,
                 float* __restrict__ weights, int ldw) {
    __shared__ float z_s[4][MOE_MAX_EXPERTS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const int t = blockIdx.x * 4 + wave;
    if (t >= n_tokens) return;               // the whole wavefront leaves; no workgroup barrier below
    float* z = z_s[threadIdx.x / 64];
    const T* hr = h + static_cast<size_t>(t) * ldh;
    for (int e = 0; e < E; ++e) {
        const float* wr = w + static_cast<size_t>(e) * D;
        float acc = 0.f;
        for (int i = lane; i < D; i += 64) acc = fmaf(wr[i], to_float(hr[i]), acc);
        acc = wave_sum(acc);
        if (lane == 0) z[e] = acc;
    }
    wave_lds_sync();
    // softmax over the experts: every lane walks all of them (E is small)
    float m = -INFINITY;
    for (int e = 0; e < E; ++e) m = fmaxf(m, z[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(z[e] - m);
    // lane e (and e + 64, ...) owns expert e: its rank is the number of experts that come before it
    for (int e = lane; e < E; e += 64) {
        const float mine = z[e];
        int before = 0;
        for (int o = 0; o < E; ++o) before += (z[o] > mine || (z[o] == mine && o < e)) ? 1 : 0;
        weights[static_cast<size_t>(t) * ldw + e] = before < top ? scale * (expf(mine - m) / sum) : 0.f;
    }
}

// out[t, e * ff + j] = weights[t, e] * relu(up[t, e * ff + j])^2 for the E experts, and behind them
// out[t, E * ff + j] = relu(up[t, E * ff + j])^2 for the shared expert's shared_ff columns.
template <typename T>
__global__ void moe_act_kernel(const T* __restrict__ up, int ldu, const float* __restrict__ weights, int ldw, int E, int ff, int N,
                               T* __restrict__ out, int ldo, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / N;
    const int c = static_cast<int>(i % N);
    const int e = c / ff;
    const float wt = e < E ? weights[t * ldw + e] : 1.f;
    const float u = fmaxf(to_float(up[t * ldu + c]), 0.f);
    out[t * ldo + c] = from_float<T>(wt * (u * u));
}

}  // namespace

extern "C" {

// h [T, D] in `dtype` (row stride ldh), w [E, D] fp32, weights [T, E] fp32 (row stride ldw).
// -1: more experts than the kernel holds, or a `top` outside 1..E.
int mllm_moe_route(const void* h, int ldh, int dtype, const float* w, int T, int D, int E, int top, float scale, float* weights, int ldw,
                   hipStream_t stream) {
    if (T <= 0) return 0;
    if (E < 1 || E > MOE_MAX_EXPERTS || top < 1 || top > E || D < 1) return -1;
    const int blocks = (T + 3) / 4;
    if (dtype == MLLM_F32) moe_route_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(h), ldh, w, T, D, E, top, scale, weights, ldw);
    else moe_route_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(h), ldh, w, T, D, E, top, scale, weights, ldw);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// up and out [T, E * ff + shared_ff] in `dtype` (out may be up).
int mllm_moe_act(const void* up, int ldu, const float* weights, int ldw, int E, int ff, int shared_ff, void* out, int ldo, int T, int dtype,
                 hipStream_t stream) {
    if (T <= 0) return 0;
    if (E < 0 || ff < 1 || shared_ff < 0 || (E > 0 && weights == nullptr)) return -1;
    const int N = E * ff + shared_ff;
    const long long total = static_cast<long long>(T) * N;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32)
        moe_act_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(up), ldu, weights, ldw, E, ff, N, static_cast<float*>(out), ldo, total);
    else
        moe_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(up), ldu, weights, ldw, E, ff, N, static_cast<bf16_t*>(out), ldo, total);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
