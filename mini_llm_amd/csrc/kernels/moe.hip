// A mixture of small feed-forward experts, for gfx950: the choice of experts and the activation between the experts'
// two products. Softmax and weights are fp32 whatever the activation dtype; the router's logits come from a product
// with fp32 results.
//
// The experts' first products are one joined product (rows [expert 0 | expert 1 | ... | shared expert]); the
// activation kernel squares the rectified values and multiplies every expert's block by the token's weight for that
// expert (zero for an expert that was not chosen, one for the shared expert), so that the experts' second products are
// one joined product as well: sum_e w_e W_down,e a_e = [W_down,0 | W_down,1 | ...] [w_0 a_0; w_1 a_1; ...].
// A second kernel serves experts that are gated and clamped, chosen by sigmoid or softmax scores, whose weight may
// stand on the expert's input, beside a shared expert that a sigmoid of the input scales.
#include "common.h"

#define MOE_MAX_EXPERTS 256

namespace {

// The weights of a token's experts from its router logits z (in LDS, E of them): scores softmax(z) over all experts,
// the `top` largest chosen (the lower index wins a tie), wgt[e] = scale * score_e for them and 0 for the others.
// Thread e < E works out expert e's weight; the caller has a barrier before (z complete) and puts one behind.
// With `sigmoid` the scores are sigmoid(z), every expert's on its own (the order of the scores is the logits' either way).
__device__ __forceinline__ void expert_weight(const float* z, float* wgt, int E, int top, float scale, int e, bool sigmoid = false) {
    const float mine = z[e];
    float m = -INFINITY;
    for (int o = 0; o < E; ++o) m = fmaxf(m, z[o]);
    float sum = 0.f;
    int before = 0;
    for (int o = 0; o < E; ++o) {
        sum += expf(z[o] - m);
        before += (z[o] > mine || (z[o] == mine && o < e)) ? 1 : 0;
    }
    const float score = sigmoid ? 1.f / (1.f + expf(-mine)) : expf(mine - m) / sum;
    wgt[e] = before < top ? scale * score : 0.f;
}

// The same for experts that are gated and clamped: the joined first product's rows are [expert 0: gate | up] ...
// [expert E-1: gate | up] [shared: gate | up], and with g = min(w G, limit), u = clamp(w U, -limit, limit) (the weight
// on the expert's INPUT, which a linear map hands on to its result; `weight_on_input` 0: g and u unweighted and the
// weight on the result) out[t, e * ff + j] = g sigmoid(alpha g) (u + 1), zero for an expert that was not chosen. The
// shared expert's columns follow, unweighted, with its own limit, times sigmoid(logits[t, E]) if `shared_gate` (the
// router's product then has one more row). One workgroup per token. VEC: eight columns a thread at a time (16-byte
// loads of bfloat16, two of float; ff, shared_ff and the strides are then multiples of 8 and the rows aligned), all of
// one expert.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_glu_act_kernel(const T* __restrict__ up, int ldu, const float* __restrict__ logits, int ldl, int E, int ff, int shared_ff, int top,
                   float scale, int sigmoid_router, float limit, float shared_limit, float alpha, int weight_on_input, int shared_gate,
                   T* __restrict__ out, int ldo) {
    __shared__ float z[MOE_MAX_EXPERTS], wgt[MOE_MAX_EXPERTS];
    __shared__ float sg_s;
    const int t = blockIdx.x, tid = threadIdx.x;
    if (tid < E) z[tid] = logits[static_cast<size_t>(t) * ldl + tid];
    if (tid == 0) sg_s = shared_gate ? 1.f / (1.f + expf(-logits[static_cast<size_t>(t) * ldl + E])) : 1.f;
    __syncthreads();
    if (tid < E) expert_weight(z, wgt, E, top, scale, tid, sigmoid_router != 0);
    __syncthreads();
    const T* ur = up + static_cast<size_t>(t) * ldu;
    T* orow = out + static_cast<size_t>(t) * ldo;
    const int routed = E * ff, N = routed + shared_ff;
    if (VEC) {
        for (int c = tid * 8; c < N; c += 256 * 8) {
            float g[8], u[8], lim, w_in = 1.f, w_out = 1.f;
            bool live = true;
            if (c < routed) {
                const int e = c / ff, j = c - e * ff;
                load8(ur + static_cast<size_t>(e) * 2 * ff + j, g);
                load8(ur + static_cast<size_t>(e) * 2 * ff + ff + j, u);
                lim = limit;
                live = wgt[e] != 0.f;
                if (weight_on_input) w_in = wgt[e]; else w_out = wgt[e];
            } else {
                const int j = c - routed;
                load8(ur + static_cast<size_t>(routed) * 2 + j, g);
                load8(ur + static_cast<size_t>(routed) * 2 + shared_ff + j, u);
                lim = shared_limit;
                w_out = sg_s;
            }
            float y[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float gk = fminf(g[k] * w_in, lim), uk = fminf(fmaxf(u[k] * w_in, -lim), lim);
                const float ex = sizeof(T) == 2 ? __expf(-alpha * gk) : expf(-alpha * gk);
                y[k] = live ? gk / (1.f + ex) * (uk + 1.f) * w_out : 0.f;
            }
            if (sizeof(T) == 2) {
                uint4 pk;
                pk.x = pack_bf16x2(y[0], y[1]); pk.y = pack_bf16x2(y[2], y[3]); pk.z = pack_bf16x2(y[4], y[5]); pk.w = pack_bf16x2(y[6], y[7]);
                *reinterpret_cast<uint4*>(orow + c) = pk;
            } else {
                *reinterpret_cast<float4*>(orow + c) = make_float4(y[0], y[1], y[2], y[3]);
                *reinterpret_cast<float4*>(orow + c + 4) = make_float4(y[4], y[5], y[6], y[7]);
            }
        }
        return;
    }
    for (int c = tid; c < N; c += 256) {
        float g, u, lim, w_in = 1.f, w_out = 1.f;
        bool live = true;
        if (c < routed) {
            const int e = c / ff, j = c - e * ff;
            g = to_float(ur[static_cast<size_t>(e) * 2 * ff + j]);
            u = to_float(ur[static_cast<size_t>(e) * 2 * ff + ff + j]);
            lim = limit;
            live = wgt[e] != 0.f;
            if (weight_on_input) w_in = wgt[e]; else w_out = wgt[e];
        } else {
            const int j = c - routed;
            g = to_float(ur[static_cast<size_t>(routed) * 2 + j]);
            u = to_float(ur[static_cast<size_t>(routed) * 2 + shared_ff + j]);
            lim = shared_limit;
            w_out = sg_s;
        }
        g = fminf(g * w_in, lim);
        u = fminf(fmaxf(u * w_in, -lim), lim);
        const float y = g / (1.f + expf(-alpha * g)) * (u + 1.f) * w_out;
        orow[c] = from_float<T>(live ? y : 0.f);
    }
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

// up [T, 2 (E * ff + shared_ff)] and out [T, E * ff + shared_ff] in `dtype`; logits [T, E (+ 1 with shared_gate)] fp32.
// -1: more experts than the kernel holds, a `top` outside 1..E, limits that are not positive.
int mllm_moe_glu_act(const void* up, int ldu, const float* logits, int ldl, int E, int ff, int shared_ff, int top, float scale,
                     int sigmoid_router, float limit, float shared_limit, float alpha, int weight_on_input, int shared_gate, void* out,
                     int ldo, int T, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (E < 1 || E > MOE_MAX_EXPERTS || top < 1 || top > E || ff < 1 || shared_ff < 0 || logits == nullptr) return -1;
    if (!(limit > 0.f) || (shared_ff > 0 && !(shared_limit > 0.f)) || (shared_gate && shared_ff == 0)) return -1;
    const int esz = dtype == MLLM_F32 ? 4 : 2;
    const bool vec = ff % 8 == 0 && shared_ff % 8 == 0 && ldu % 8 == 0 && ldo % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 && (static_cast<size_t>(ldu) * esz) % 16 == 0;
#define MOE_GLU(TYPE, VEC)                                                                                                                     \
    moe_glu_act_kernel<TYPE, VEC><<<T, 256, 0, stream>>>(static_cast<const TYPE*>(up), ldu, logits, ldl, E, ff, shared_ff, top, scale, sigmoid_router, \
                                                         limit, shared_limit, alpha, weight_on_input, shared_gate, static_cast<TYPE*>(out), ldo)
    if (dtype == MLLM_F32) { if (vec) MOE_GLU(float, true); else MOE_GLU(float, false); }
    else { if (vec) MOE_GLU(bf16_t, true); else MOE_GLU(bf16_t, false); }
#undef MOE_GLU
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
