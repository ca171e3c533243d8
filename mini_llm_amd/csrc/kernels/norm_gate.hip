// RMS norms (plain, grouped, gated), the normed and scaled residual add, the clamped gated activation
// and a fill, for gfx950. Statistics and sums are fp32 whatever the activation dtype.
#include <algorithm>

#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_precise(float v) { return 1.f / (1.f + expf(-v)); }

// One wavefront per (row, group): y[r, g*Dg + i] = v_i / sqrt(mean_i(v_i^2) + eps) * w[g*Dg + i], with
// v = x[src row, g*Dg + i] (times silu(gate[row, g*Dg + i]) when a gate is given: the gate comes before
// the norm). `rows` (optional) selects the input rows. WAVES (row, group) pairs per workgroup.
template <typename OutT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_kernel(const float* __restrict__ x, int ldx, const int* __restrict__ rows, const float* __restrict__ w,
               const float* __restrict__ gate, int ldg, OutT* __restrict__ y, int ldy, int n, int D, int groups,
               float eps, int parts, size_t part_stride) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const long long pair = static_cast<long long>(blockIdx.x) * WAVES + wave;
    if (pair >= static_cast<long long>(n) * groups) return;
    const int r = static_cast<int>(pair / groups), g = static_cast<int>(pair % groups), Dg = D / groups;
    const int src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * ldx + g * Dg;
    auto input = [&](int i) {
        float a = xr[i];
        for (int part = 1; part < parts; ++part) a += xr[part * part_stride + i];
        return a;
    };
    const float* gr = gate ? gate + static_cast<size_t>(src) * ldg + g * Dg : nullptr;
    const float* wr = w + g * Dg;
    OutT* yr = y + static_cast<size_t>(r) * ldy + g * Dg;
    // up to 8 elements a lane stay in registers; longer rows are read again
    float v[8];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        float a = 0.f;
        if (i < Dg) {
            a = input(i);
            if (gr) { const float z = gr[i]; a *= z * sigmoid_precise(z); }
        }
        v[u] = a;
        ss += a * a;
    }
    for (int i = lane + 512; i < Dg; i += 64) {
        float a = input(i);
        if (gr) { const float z = gr[i]; a *= z * sigmoid_precise(z); }
        ss += a * a;
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dg) + eps);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (i < Dg) yr[i] = from_float<OutT>(v[u] * inv * wr[i]);
    }
    for (int i = lane + 512; i < Dg; i += 64) {
        float a = input(i);
        if (gr) { const float z = gr[i]; a *= z * sigmoid_precise(z); }
        yr[i] = from_float<OutT>(a * inv * wr[i]);
    }
}


// One wavefront per (row, group): y[r, g*Dg + i] = v_i / sqrt(mean_i(v_i^2) + eps) * w[g*Dg + i] * silu(gate[r, g*Dg + i]),
// the gate BEHIND the norm (w may be null: no weight). v is the sum of `parts` arrays part_stride floats apart, added
// in the order of their index. The heads of a linear-attention mixer, normed one by one and gated.
template <typename OutT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_gate_after_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ gate, int ldg,
                          OutT* __restrict__ y, int ldy, int n, int D, int groups, float eps, int parts, size_t part_stride) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const long long pair = static_cast<long long>(blockIdx.x) * WAVES + wave;
    if (pair >= static_cast<long long>(n) * groups) return;
    const int r = static_cast<int>(pair / groups), g = static_cast<int>(pair % groups), Dg = D / groups;
    const float* xr = x + static_cast<size_t>(r) * ldx + g * Dg;
    const float* gr = gate + static_cast<size_t>(r) * ldg + g * Dg;
    OutT* yr = y + static_cast<size_t>(r) * ldy + g * Dg;
    // up to 4 elements a lane stay in registers (heads of up to 256 columns); longer groups are read again
    float v[4], z[4], ww[4];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = min(lane + 64 * u, Dg - 1);
        float a = xr[i];
        for (int part = 1; part < parts; ++part) a += xr[part * part_stride + i];
        v[u] = a;
        z[u] = gr[i];
        ww[u] = w ? w[g * Dg + i] : 1.f;
        if (lane + 64 * u < Dg) ss += a * a;
    }
    for (int i = lane + 256; i < Dg; i += 64) {
        float a = xr[i];
        for (int part = 1; part < parts; ++part) a += xr[part * part_stride + i];
        ss += a * a;
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dg) + eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = lane + 64 * u;
        if (i < Dg) yr[i] = from_float<OutT>(v[u] * inv * ww[u] * (z[u] * sigmoid_precise(z[u])));
    }
    for (int i = lane + 256; i < Dg; i += 64) {
        float a = xr[i];
        for (int part = 1; part < parts; ++part) a += xr[part * part_stride + i];
        const float zz = gr[i];
        yr[i] = from_float<OutT>(a * inv * (w ? w[g * Dg + i] : 1.f) * (zz * sigmoid_precise(zz)));
    }
}

// out[i] = cap * tanh(x[i] / cap), in place (fp32)
__global__ void softcap_kernel(float* __restrict__ x, float cap, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// x[r, i] += mult * scale[i] * (y[r, i] / sqrt(mean(y[r]^2) + eps) * w[i]); one wavefront per row.
// With `clear` the row of y is set to zero behind the read, ready to collect the next sub-layer's output.
template <int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_add_kernel(float* __restrict__ y, const float* __restrict__ w, const float* __restrict__ scale, float mult,
                   float eps, float* __restrict__ x, int n, int D, int clear) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int r = blockIdx.x * WAVES + wave;
    if (r >= n) return;
    float* yr = y + static_cast<size_t>(r) * D;
    float* xr = x + static_cast<size_t>(r) * D;
    float v[8];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        v[u] = i < D ? yr[i] : 0.f;
        ss += v[u] * v[u];
    }
    for (int i = lane + 512; i < D; i += 64) ss += yr[i] * yr[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + eps);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (i < D) {
            const float s = scale ? scale[i] * mult : mult;
            xr[i] += s * (v[u] * inv * w[i]);
            if (clear) yr[i] = 0.f;
        }
    }
    for (int i = lane + 512; i < D; i += 64) {
        const float s = scale ? scale[i] * mult : mult;
        xr[i] += s * (yr[i] * inv * w[i]);
        if (clear) yr[i] = 0.f;
    }
}

// Many short groups (heads of a recurrence: 16 to 128 columns each): LANES = columns / 4 lanes take one (row, group)
// pair, a wavefront 64 / LANES of them, so that every lane holds four columns whatever the group's size (one wavefront
// per pair leaves 48 of 64 lanes idle at 64 columns). Up to four shares are added in the order of their index; no
// gate, no row selection. All loads without conditions, from clamped places.
template <typename OutT, int LANES>
__global__ void __launch_bounds__(256)
rmsnorm_small_groups_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, OutT* __restrict__ y, int ldy,
                            long long pairs, int groups, float eps, int parts, size_t part_stride) {
    constexpr int PER_WAVE = 64 / LANES, DG = 4 * LANES;
    const int lane = threadIdx.x % MLLM_WAVE, sub = lane % LANES;
    const long long wave = static_cast<long long>(blockIdx.x) * 4 + threadIdx.x / MLLM_WAVE;
    const long long mine = wave * PER_WAVE + lane / LANES;
    const bool valid = mine < pairs;
    const long long pair = valid ? mine : pairs - 1;
    const long long r = pair / groups;
    const int g = static_cast<int>(pair % groups);
    const float* xr = x + static_cast<size_t>(r) * ldx + g * DG + 4 * sub;
    float4 v = *reinterpret_cast<const float4*>(xr);
    float4 sh[3];
#pragma unroll
    for (int part = 1; part < 4; ++part) sh[part - 1] = *reinterpret_cast<const float4*>(xr + min(part, parts - 1) * part_stride);
    const float4 ww = *reinterpret_cast<const float4*>(w + g * DG + 4 * sub);
#pragma unroll
    for (int part = 1; part < 4; ++part)
        if (part < parts) { v.x += sh[part - 1].x; v.y += sh[part - 1].y; v.z += sh[part - 1].z; v.w += sh[part - 1].w; }
    const float ss = group_sum<LANES>((v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w));
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(DG) + eps);
    if (!valid) return;
    OutT* yr = y + static_cast<size_t>(r) * ldy + g * DG + 4 * sub;
    const float o0 = v.x * inv * ww.x, o1 = v.y * inv * ww.y, o2 = v.z * inv * ww.z, o3 = v.w * inv * ww.w;
    if (sizeof(OutT) == 2) {
        uint2 pk;
        pk.x = pack_bf16x2(o0, o1);
        pk.y = pack_bf16x2(o2, o3);
        *reinterpret_cast<uint2*>(yr) = pk;
    } else {
        *reinterpret_cast<float4*>(yr) = make_float4(o0, o1, o2, o3);
    }
}

// x[r, i] += mult * sum_k y_k[r, i] / sqrt(mean(y_k[r]^2) + eps) * w_k[i] for n inputs of x's shape that lie
// y_stride floats apart (weights w_stride apart), added in the order of k; one wavefront per row.
// N_IN inputs, NB blocks of 512 columns: every input row stays in registers between its statistics and the sum; loads
// without conditions, from clamped places, masked where they are used.
template <int WAVES, int N_IN, int NB>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_add_many_kernel(const float* __restrict__ y, size_t y_stride, const float* __restrict__ w, size_t w_stride,
                        float mult, float eps, float* __restrict__ x, int n, int D) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int r = blockIdx.x * WAVES + wave;
    if (r >= n) return;
    float v[N_IN][NB][8], xv[NB][8];
#pragma unroll
    for (int k = 0; k < N_IN; ++k)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int u = 0; u < 8; ++u) v[k][b][u] = y[k * y_stride + static_cast<size_t>(r) * D + min(512 * b + lane + 64 * u, D - 1)];
    float* xr = x + static_cast<size_t>(r) * D;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int u = 0; u < 8; ++u) xv[b][u] = xr[min(512 * b + lane + 64 * u, D - 1)];
    float inv[N_IN];
#pragma unroll
    for (int k = 0; k < N_IN; ++k) {
        float ss = 0.f;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int u = 0; u < 8; ++u) ss += (512 * b + lane + 64 * u < D) ? v[k][b][u] * v[k][b][u] : 0.f;
        inv[k] = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + eps);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        float g[N_IN][8];
#pragma unroll
        for (int k = 0; k < N_IN; ++k)
#pragma unroll
            for (int u = 0; u < 8; ++u) g[k][u] = w[k * w_stride + min(512 * b + lane + 64 * u, D - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < N_IN; ++k) a += v[k][b][u] * inv[k] * g[k][u];
            if (512 * b + lane + 64 * u < D) xr[512 * b + lane + 64 * u] = xv[b][u] + mult * a;
        }
    }
}

// The same two norms for rows whose parts are multiples of 4 and at most 2,048 long, 16-byte aligned: the part
// lives in registers as float4, and every load is issued without a condition, from a clamped index, before the
// first use (a load under a condition waits for all loads in flight, and a row of 768 then costs eight round trips).
// `parts` > 1: the input is the sum of that many arrays `part_stride` floats apart (partial results of a kernel
// that splits a sum over workgroups), added in the order of their index.
template <typename OutT, int WAVES, bool SHARES = false>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_vec_kernel(const float* __restrict__ x, int ldx, const int* __restrict__ rows, const float* __restrict__ w,
                   const float* __restrict__ gate, int ldg, OutT* __restrict__ y, int ldy, int n, int D, int groups,
                   float eps, int parts, size_t part_stride) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const long long pair = static_cast<long long>(blockIdx.x) * WAVES + wave;
    if (pair >= static_cast<long long>(n) * groups) return;
    const int r = static_cast<int>(pair / groups), g = static_cast<int>(pair % groups), Dg = D / groups;
    const int src = rows ? rows[r] : r;
    const float4* xr = reinterpret_cast<const float4*>(x + static_cast<size_t>(src) * ldx + g * Dg);
    const float4* gr = reinterpret_cast<const float4*>(gate ? gate + static_cast<size_t>(src) * ldg + g * Dg : x);
    const float4* wr = reinterpret_cast<const float4*>(w + g * Dg);
    const int nq = Dg / 4, n_u = (nq + 63) / 64;
    float4 v[8], gg[8], ww[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) v[u] = xr[min(lane + 64 * u, nq - 1)];
    if (SHARES) {
        // up to four shares (the launcher sends more to the plain kernel): all of them requested before the first
        // is added, a share beyond `parts` read from the last one and not added
        float4 sh[3][8];
#pragma unroll
        for (int part = 1; part < 4; ++part) {
            const float4* xp = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xr) + min(part, parts - 1) * part_stride);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (u < n_u) sh[part - 1][u] = xp[min(lane + 64 * u, nq - 1)];
        }
#pragma unroll
        for (int part = 1; part < 4; ++part)
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (u < n_u && part < parts) {
                    v[u].x += sh[part - 1][u].x; v[u].y += sh[part - 1][u].y; v[u].z += sh[part - 1][u].z; v[u].w += sh[part - 1][u].w;
                }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) {
            const int i = min(lane + 64 * u, nq - 1);
            gg[u] = gr[i];
            ww[u] = wr[i];
        }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) {
            if (gate) {
                v[u].x *= gg[u].x * sigmoid_precise(gg[u].x); v[u].y *= gg[u].y * sigmoid_precise(gg[u].y);
                v[u].z *= gg[u].z * sigmoid_precise(gg[u].z); v[u].w *= gg[u].w * sigmoid_precise(gg[u].w);
            }
            if (lane + 64 * u < nq) ss += (v[u].x * v[u].x + v[u].y * v[u].y) + (v[u].z * v[u].z + v[u].w * v[u].w);
        }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dg) + eps);
    OutT* yr = y + static_cast<size_t>(r) * ldy + g * Dg;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (u < n_u && i < nq) {
            const float o0 = v[u].x * inv * ww[u].x, o1 = v[u].y * inv * ww[u].y, o2 = v[u].z * inv * ww[u].z, o3 = v[u].w * inv * ww[u].w;
            if (sizeof(OutT) == 2) {
                uint2 pk;
                pk.x = pack_bf16x2(o0, o1);
                pk.y = pack_bf16x2(o2, o3);
                *reinterpret_cast<uint2*>(yr + 4 * i) = pk;
            } else {
                *reinterpret_cast<float4*>(yr + 4 * i) = make_float4(o0, o1, o2, o3);
            }
        }
    }
}

template <int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
rmsnorm_add_vec_kernel(float* __restrict__ y, const float* __restrict__ w, const float* __restrict__ scale, float mult,
                       float eps, float* __restrict__ x, int n, int D, int clear) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int r = blockIdx.x * WAVES + wave;
    if (r >= n) return;
    float4* yr = reinterpret_cast<float4*>(y + static_cast<size_t>(r) * D);
    float4* xr = reinterpret_cast<float4*>(x + static_cast<size_t>(r) * D);
    const float4* wr = reinterpret_cast<const float4*>(w);
    const float4* sr = reinterpret_cast<const float4*>(scale ? scale : w);
    const int nq = D / 4, n_u = (nq + 63) / 64;
    float4 v[8], xx[8], ww[8], sc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) v[u] = yr[min(lane + 64 * u, nq - 1)];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) {
            const int i = min(lane + 64 * u, nq - 1);
            xx[u] = xr[i];
            ww[u] = wr[i];
            sc[u] = sr[i];
        }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u && lane + 64 * u < nq) ss += (v[u].x * v[u].x + v[u].y * v[u].y) + (v[u].z * v[u].z + v[u].w * v[u].w);
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + eps);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (u < n_u && i < nq) {
            const float4 s4 = scale ? make_float4(sc[u].x * mult, sc[u].y * mult, sc[u].z * mult, sc[u].w * mult) : make_float4(mult, mult, mult, mult);
            xr[i] = make_float4(xx[u].x + s4.x * (v[u].x * inv * ww[u].x), xx[u].y + s4.y * (v[u].y * inv * ww[u].y),
                                xx[u].z + s4.z * (v[u].z * inv * ww[u].z), xx[u].w + s4.w * (v[u].w * inv * ww[u].w));
            if (clear) yr[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
}

// out[t, i] = g sigmoid(alpha g) (u + 1) with g = min(gate[t, i], limit), u = clamp(up[t, i], -limit, limit).
template <typename T>
__global__ void glu_clamped_kernel(const T* gate, int ldg, const T* up, int ldu, T* out, int ldo,     // (out may be gate)
                                   long long total, int F, float limit, float alpha) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / F), f = static_cast<int>(i % F);
    const float g = fminf(to_float(gate[static_cast<size_t>(t) * ldg + f]), limit);
    const float u = fminf(fmaxf(to_float(up[static_cast<size_t>(t) * ldu + f]), -limit), limit);
    const float s = sizeof(T) == 4 ? sigmoid_precise(alpha * g) : __builtin_amdgcn_rcpf(1.f + __expf(-alpha * g));
    out[static_cast<size_t>(t) * ldo + f] = from_float<T>(g * s * (u + 1.f));
}

__global__ void fill_zero_kernel(float4* __restrict__ p, size_t n4) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

}  // namespace

extern "C" {

// y = rmsnorm(x[rows]) in `groups` equal parts of the D columns, optionally gated (see the kernel).
// x and gate fp32 with row strides ldx / ldg; y in out_dtype with row stride ldy. With parts > 1, x is the sum of
// `parts` arrays part_stride floats apart. -1: D is no multiple of groups.
int mllm_rmsnorm(const float* x, int ldx, const int* rows, const float* w, const float* gate, int ldg, void* y, int ldy,
                 int n, int D, int groups, float eps, int out_dtype, int parts, size_t part_stride, hipStream_t stream) {
    if (n <= 0 || D <= 0) return 0;
    if (groups < 1 || D % groups != 0 || parts < 1) return -1;
    const long long pairs = static_cast<long long>(n) * groups;
    const int Dg = D / groups, esz = out_dtype == MLLM_F32 ? 4 : 2;
    const bool vec = parts <= 4 && Dg % 4 == 0 && Dg <= 2048 && ldx % 4 == 0 && (gate == nullptr || ldg % 4 == 0) && part_stride % 4 == 0 &&
                     (static_cast<size_t>(ldy) * esz) % 16 == 0 && (static_cast<size_t>(Dg) * esz) % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(gate) |
                       reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    // (workgroups start at a limited rate: many rows go eight to a workgroup)
#define RMS(KERNEL, TYPE, WAVES)                                                                                        \
    KERNEL<TYPE, WAVES><<<static_cast<int>((pairs + WAVES - 1) / WAVES), 64 * WAVES, 0, stream>>>(                      \
        x, ldx, rows, w, gate, ldg, static_cast<TYPE*>(y), ldy, n, D, groups, eps, parts, part_stride)
#define RMS_SHARES(TYPE)                                                                                                \
    rmsnorm_vec_kernel<TYPE, 4, true><<<static_cast<int>((pairs + 3) / 4), 256, 0, stream>>>(                           \
        x, ldx, rows, w, gate, ldg, static_cast<TYPE*>(y), ldy, n, D, groups, eps, parts, part_stride)
    if (vec && groups > 1 && rows == nullptr && gate == nullptr && (Dg == 16 || Dg == 32 || Dg == 64 || Dg == 128)) {
        // many short groups: several of them a wavefront
        const int per_wg = 4 * (64 / (Dg / 4));
        const int blocks = static_cast<int>((pairs + per_wg - 1) / per_wg);
#define RSG(TYPE, LANES)                                                                                              \
    rmsnorm_small_groups_kernel<TYPE, LANES><<<blocks, 256, 0, stream>>>(x, ldx, w, static_cast<TYPE*>(y), ldy, pairs, groups, eps, parts, \
                                                                        part_stride)
#define RSG_T(TYPE) do { if (Dg == 16) RSG(TYPE, 4); else if (Dg == 32) RSG(TYPE, 8); else if (Dg == 64) RSG(TYPE, 16); else RSG(TYPE, 32); } while (0)
        if (out_dtype == MLLM_F32) RSG_T(float); else RSG_T(bf16_t);
#undef RSG_T
#undef RSG
    } else if (vec && parts > 1) {
        if (out_dtype == MLLM_F32) RMS_SHARES(float); else RMS_SHARES(bf16_t);
    } else if (vec) {
        if (out_dtype == MLLM_F32) { if (pairs >= 512) RMS(rmsnorm_vec_kernel, float, 8); else RMS(rmsnorm_vec_kernel, float, 4); }
        else { if (pairs >= 512) RMS(rmsnorm_vec_kernel, bf16_t, 8); else RMS(rmsnorm_vec_kernel, bf16_t, 4); }
    } else {
        if (out_dtype == MLLM_F32) RMS(rmsnorm_kernel, float, 4); else RMS(rmsnorm_kernel, bf16_t, 4);
    }
#undef RMS
#undef RMS_SHARES
    MLLM_LAUNCH_CHECK();
    return 0;
}

// y = rmsnorm(x) * w * silu(gate) in `groups` equal parts of the D columns, the gate behind the norm; w ([D]) may be
// null. x and gate fp32 with row strides ldx / ldg; with parts > 1, x is the sum of `parts` arrays part_stride floats
// apart. -1: D is no multiple of groups.
int mllm_rmsnorm_gate_after(const float* x, int ldx, const float* w, const float* gate, int ldg, void* y, int ldy, int n, int D, int groups,
                            float eps, int out_dtype, int parts, size_t part_stride, hipStream_t stream) {
    if (n <= 0 || D <= 0) return 0;
    if (groups < 1 || D % groups != 0 || parts < 1 || gate == nullptr) return -1;
    const long long pairs = static_cast<long long>(n) * groups;
    const int blocks = static_cast<int>((pairs + 3) / 4);
    if (out_dtype == MLLM_F32)
        rmsnorm_gate_after_kernel<float, 4><<<blocks, 256, 0, stream>>>(x, ldx, w, gate, ldg, static_cast<float*>(y), ldy, n, D, groups, eps, parts, part_stride);
    else
        rmsnorm_gate_after_kernel<bf16_t, 4><<<blocks, 256, 0, stream>>>(x, ldx, w, gate, ldg, static_cast<bf16_t*>(y), ldy, n, D, groups, eps, parts, part_stride);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// x <- cap tanh(x / cap) over n contiguous floats. -1: a cap that is not positive.
int mllm_softcap(float* x, size_t n, float cap, hipStream_t stream) {
    if (n == 0) return 0;
    if (!(cap > 0.f)) return -1;
    softcap_kernel<<<static_cast<int>((n + 255) / 256), 256, 0, stream>>>(x, cap, n);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_rmsnorm_add(float* y, const float* w, const float* scale, float mult, float eps, float* x, int n, int D,
                     int clear, hipStream_t stream) {
    if (n <= 0 || D <= 0) return 0;
    const bool vec = D % 4 == 0 && D <= 2048 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(scale) |
                       reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (vec && n >= 512) rmsnorm_add_vec_kernel<8><<<(n + 7) / 8, 512, 0, stream>>>(y, w, scale, mult, eps, x, n, D, clear);
    else if (vec) rmsnorm_add_vec_kernel<4><<<(n + 3) / 4, 256, 0, stream>>>(y, w, scale, mult, eps, x, n, D, clear);
    else rmsnorm_add_kernel<4><<<(n + 3) / 4, 256, 0, stream>>>(y, w, scale, mult, eps, x, n, D, clear);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// -1: fewer than 2 or more than 4 inputs, or rows of more than 2,048 columns
int mllm_rmsnorm_add_many(const float* y, size_t y_stride, const float* w, size_t w_stride, int n_in, float mult, float eps,
                          float* x, int n, int D, hipStream_t stream) {
    if (n <= 0 || D <= 0) return 0;
    if (n_in < 2 || n_in > 4 || D > 2048) return -1;
#define RAM(N_IN, NB)                                                                                                  \
    do {                                                                                                               \
        if (n >= 512) rmsnorm_add_many_kernel<8, N_IN, NB><<<(n + 7) / 8, 512, 0, stream>>>(y, y_stride, w, w_stride, mult, eps, x, n, D); \
        else rmsnorm_add_many_kernel<4, N_IN, NB><<<(n + 3) / 4, 256, 0, stream>>>(y, y_stride, w, w_stride, mult, eps, x, n, D); \
    } while (0)
#define RAM_NB(N_IN) do { if (D <= 512) RAM(N_IN, 1); else if (D <= 1024) RAM(N_IN, 2); else RAM(N_IN, 4); } while (0)
    if (n_in == 2) RAM_NB(2); else if (n_in == 3) RAM_NB(3); else RAM_NB(4);
#undef RAM_NB
#undef RAM
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_glu_clamped(const void* gate, int ldg, const void* up, int ldu, void* out, int ldo, int T, int F, float limit,
                     float alpha, int dtype, hipStream_t stream) {
    if (T <= 0 || F <= 0) return 0;
    const long long total = static_cast<long long>(T) * F;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32)
        glu_clamped_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(gate), ldg, static_cast<const float*>(up), ldu,
                                                              static_cast<float*>(out), ldo, total, F, limit, alpha);
    else
        glu_clamped_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(gate), ldg, static_cast<const bf16_t*>(up), ldu,
                                                               static_cast<bf16_t*>(out), ldo, total, F, limit, alpha);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// Clears `bytes` bytes (a multiple of 16, the address 16-byte aligned; -1 otherwise) with a kernel, so that
// the call may be captured into a graph.
int mllm_fill_zero(void* p, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return 0;
    if (bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    const size_t n4 = bytes / 16;
    const int blocks = static_cast<int>(std::min<size_t>((n4 + 255) / 256, 2048));
    fill_zero_kernel<<<blocks, 256, 0, stream>>>(static_cast<float4*>(p), n4);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
