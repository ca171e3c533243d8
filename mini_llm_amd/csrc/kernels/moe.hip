// A mixture of small feed-forward experts, for gfx950: the choice of experts and the activation between the experts'
// two products. Softmax and weights are fp32 whatever the activation dtype; the router's logits come from a product
// with fp32 results.
//
// The experts' first products are one joined product (rows [expert 0 | expert 1 | ... | shared expert]); the
// activation kernel squares the rectified values and multiplies every expert's block by the token's weight for that
// expert (zero for an expert that was not chosen, one for the shared expert), so that the experts' second products are
// one joined product as well: sum_e w_e W_down,e a_e = [W_down,0 | W_down,1 | ...] [w_0 a_0; w_1 a_1; ...].
#include "common.h"

#define MOE_MAX_EXPERTS 256

namespace {

// The weights of a token's experts from its router logits z (in LDS, E of them): scores softmax(z) over all experts,
// the `top` largest chosen (the lower index wins a tie), wgt[e] = scale * score_e for them and 0 for the others.
// Thread e < E works out expert e's weight; the caller has a barrier before (z complete) and puts one behind.
__device__ __forceinline__ void expert_weight(const float* z, float* wgt, int E, int top, float scale, int e) {
    const float mine = z[e];
    float m = -INFINITY;
    for (int o = 0; o < E; ++o) m = fmaxf(m, z[o]);
    float sum = 0.f;
    int before = 0;
    for (int o = 0; o < E; ++o) {
        sum += expf(z[o] - m);
        before += (z[o] > mine || (z[o] == mine && o < e)) ? 1 : 0;
    }
    wgt[e] = before < top ? scale * (expf(mine - m) / sum) : 0.f;
}

// One workgroup per token: the weights from the token's logits, then
// out[t, e * ff + j] = weight_e * relu(up[t, e * ff + j])^2 for the E experts, and behind them
// out[t, E * ff + j] = relu(up[t, E * ff + j])^2 for the shared expert's columns (N columns in all).
// VEC: eight columns a thread at a time (16-byte loads of bfloat16, two of float; ff, N and the strides are then
// multiples of 8 and the rows aligned). `weights_out` (optional, [T, E]) receives the weights.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_act_kernel(const T* __restrict__ up, int ldu, const float* __restrict__ logits, int ldl, int E, int ff, int N, int top, float scale,
               T* __restrict__ out, int ldo, float* __restrict__ weights_out, int ldw) {
    __shared__ float z[MOE_MAX_EXPERTS], wgt[MOE_MAX_EXPERTS];
    const int t = blockIdx.x, tid = threadIdx.x;
    if (tid < E) z[tid] = logits[static_cast<size_t>(t) * ldl + tid];
    __syncthreads();
    if (tid < E) {
        expert_weight(z, wgt, E, top, scale, tid);
        if (weights_out != nullptr) weights_out[static_cast<size_t>(t) * ldw + tid] = wgt[tid];
    }
    __syncthreads();
    const T* ur = up + static_cast<size_t>(t) * ldu;
    T* orow = out + static_cast<size_t>(t) * ldo;
    if (VEC) {
        for (int c = tid * 8; c < N; c += 256 * 8) {
            float v[8];
            load8(ur + c, v);
            const int e = c / ff;                       // (ff is a multiple of 8: the eight columns are one expert's)
            const float wt = e < E ? wgt[e] : 1.f;
#pragma unroll
            for (int u = 0; u < 8; ++u) { const float r = fmaxf(v[u], 0.f); v[u] = wt * (r * r); }
            if (sizeof(T) == 2) {
                uint4 pk;
                pk.x = pack_bf16x2(v[0], v[1]); pk.y = pack_bf16x2(v[2], v[3]); pk.z = pack_bf16x2(v[4], v[5]); pk.w = pack_bf16x2(v[6], v[7]);
                *reinterpret_cast<uint4*>(orow + c) = pk;
            } else {
                *reinterpret_cast<float4*>(orow + c) = make_float4(v[0], v[1], v[2], v[3]);
                *reinterpret_cast<float4*>(orow + c + 4) = make_float4(v[4], v[5], v[6], v[7]);
            }
        }
    } else {
        for (int c = tid; c < N; c += 256) {
            const int e = c / ff;
            const float wt = e < E ? wgt[e] : 1.f;
            const float r = fmaxf(to_float(ur[c]), 0.f);
            orow[c] = from_float<T>(wt * (r * r));
        }
    }
}

}  // namespace

extern "C" {

// up and out [T, E * ff + shared_ff] in `dtype` (out may be up); logits [T, E] fp32 (row stride ldl); weights_out
// (optional) [T, E] fp32. -1: more experts than the kernel holds, or a `top` outside 1..E.
int mllm_moe_act(const void* up, int ldu, const float* logits, int ldl, int E, int ff, int shared_ff, int top, float scale, void* out, int ldo,
                 float* weights_out, int ldw, int T, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (E < 1 || E > MOE_MAX_EXPERTS || top < 1 || top > E || ff < 1 || shared_ff < 0 || logits == nullptr) return -1;
    const int N = E * ff + shared_ff;
    const int esz = dtype == MLLM_F32 ? 4 : 2;
    const bool vec = ff % 8 == 0 && N % 8 == 0 && ldu % 8 == 0 && ldo % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 && (static_cast<size_t>(ldu) * esz) % 16 == 0;
#define MOE_ACT(TYPE, VEC)                                                                                                          \
    moe_act_kernel<TYPE, VEC><<<T, 256, 0, stream>>>(static_cast<const TYPE*>(up), ldu, logits, ldl, E, ff, N, top, scale,           \
                                                     static_cast<TYPE*>(out), ldo, weights_out, ldw)
    if (dtype == MLLM_F32) { if (vec) MOE_ACT(float, true); else MOE_ACT(float, false); }
    else { if (vec) MOE_ACT(bf16_t, true); else MOE_ACT(bf16_t, false); }
#undef MOE_ACT
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
