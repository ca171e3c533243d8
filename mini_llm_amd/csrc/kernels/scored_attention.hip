// Softmax attention over the paged cache whose scores are shaped before the softmax, for gfx950:
//   s = scale (q . k);  s <- cap tanh(s / cap) (cap > 0);  s <- s - r1[h] ln(1 + r2[h] (i - j)) (a distance bias per head)
// under a causal mask that is plain, a sliding window (0 <= i - j < window) or chunked (j <= i within the
// chunk of `chunk` positions that holds i, chunks counted from position 0), with value rows of a width of
// their own and an optional sigmoid gate on the result. Scores, softmax and the value sum are fp32.
//
// Before it, `qk_prepare` makes queries, keys and values ready from the rows of the input projection: an
// RMS norm of queries and keys (per head with one weight shared by the heads, or over the whole row), a
// rotation of the first rot_dims columns of every head in the half-split layout (column i pairs with
// i + rot_dims / 2) or the interleaved one (column 2i pairs with 2i + 1), optionally a scaling of every head to unit
// root mean square behind the rotation (no weight), and the write of the keys and values to their page rows.
// The scores may also carry a linear distance bias per head, the softmax one more term exp(sink[h]) in its
// denominator, and a sliding window may keep the sequence's first positions visible.
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_of(float v) { return 1.f / (1.f + expf(-v)); }

enum NormMode : int { NORM_NONE = 0, NORM_HEAD = 1, NORM_ROW = 2, NORM_UNIT_AFTER = 3 };

// The partner of column i among the first rot_dims columns, the index of the pair's angle, and whether i is the
// pair's first column: half-split (i, i + rot_dims / 2) or interleaved (2i, 2i + 1).
__device__ __forceinline__ int rot_partner(int i, int half, bool interleaved) { return interleaved ? (i ^ 1) : (i < half ? i + half : i - half); }
__device__ __forceinline__ int rot_pair(int i, int half, bool interleaved) { return interleaved ? i / 2 : (i < half ? i : i - half); }
__device__ __forceinline__ bool rot_first(int i, int half, bool interleaved) { return interleaved ? (i & 1) == 0 : i < half; }

// One workgroup per token. proj row (fp32): queries at q_col (H heads of d), keys at k_col (G heads of d), values at
// v_col (G heads of dv; v_col < 0: the values are the keys as projected, before their norm; then dv == d).
// LDS: the query and key rows, cos/sin of the token's angles, the inverse root mean squares.
template <typename T>
__global__ void __launch_bounds__(256)
qk_prepare_kernel(const float* __restrict__ proj, int ld, int q_col, int k_col, int v_col, int H, int G, int d, int dv,
                  int norm_mode, const float* __restrict__ wq, const float* __restrict__ wk, float eps, int rot_dims,
                  double rot_base, int interleaved, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ q_out,
                  int ldq, T* __restrict__ k_pages, T* __restrict__ v_pages) {
    extern __shared__ float pr_smem[];
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int nq = H * d, nk = G * d, half = rot_dims / 2;
    float* qs = pr_smem;                 // [nq]
    float* ks = qs + nq;                 // [nk]
    float* cs = ks + nk;                 // [half] cos, [half] sin
    float* inv = cs + 2 * half;          // [H + G] (head mode) or [2] (row mode)
    __shared__ float red[16];
    const float* row = proj + static_cast<size_t>(t) * ld;
    for (int i = tid; i < nq; i += 256) qs[i] = row[q_col + i];
    for (int i = tid; i < nk; i += 256) ks[i] = row[k_col + i];
    if (tid < half) {
        // the angle in double, rounded once
        const double f = pow(rot_base, -2.0 * tid / rot_dims), a = static_cast<double>(positions[t]) * f;
        cs[tid] = static_cast<float>(cos(a));
        cs[half + tid] = static_cast<float>(sin(a));
    }
    __syncthreads();
    if (norm_mode == NORM_HEAD) {
        for (int h = wave; h < H + G; h += 4) {
            const float* v = h < H ? qs + h * d : ks + (h - H) * d;
            float ss = 0.f;
            for (int i = lane; i < d; i += 64) ss += v[i] * v[i];
            ss = wave_sum(ss);
            if (lane == 0) inv[h] = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
        }
    } else if (norm_mode == NORM_ROW) {
        float ss = 0.f;
        for (int i = tid; i < nq; i += 256) ss += qs[i] * qs[i];
        const float sq = block_sum(ss, red);
        ss = 0.f;
        for (int i = tid; i < nk; i += 256) ss += ks[i] * ks[i];
        const float sk = block_sum(ss, red);
        if (tid == 0) {
            inv[0] = 1.0f / sqrtf(sq / static_cast<float>(nq) + eps);
            inv[1] = 1.0f / sqrtf(sk / static_cast<float>(nk) + eps);
        }
    }
    __syncthreads();
    const int slot = slots != nullptr ? slots[t] : -1;
    const bool il = interleaved != 0;
    // the normed value of column i of head h of the queries (is_k: of the keys)
    auto normed = [&](bool is_k, int h, int i) {
        const float raw = is_k ? ks[h * d + i] : qs[h * d + i];
        if (norm_mode == NORM_NONE || norm_mode == NORM_UNIT_AFTER) return raw;
        if (norm_mode == NORM_HEAD) return raw * inv[is_k ? H + h : h] * (is_k ? wk[i] : wq[i]);
        return raw * inv[is_k ? 1 : 0] * (is_k ? wk[h * d + i] : wq[h * d + i]);
    };
    auto turned_plain = [&](bool is_k, int h, int i) {
        const float a = normed(is_k, h, i);
        if (i >= rot_dims) return a;
        const int pi = rot_pair(i, half, il);
        const float b = normed(is_k, h, rot_partner(i, half, il));
        return rot_first(i, half, il) ? a * cs[pi] - b * cs[half + pi] : a * cs[pi] + b * cs[half + pi];
    };
    if (norm_mode == NORM_UNIT_AFTER) {
        // every head's root mean square behind the rotation
        for (int h = wave; h < H + G; h += 4) {
            const bool is_k = h >= H;
            float ss = 0.f;
            for (int i = lane; i < d; i += 64) { const float v = turned_plain(is_k, is_k ? h - H : h, i); ss += v * v; }
            ss = wave_sum(ss);
            if (lane == 0) inv[h] = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
        }
        __syncthreads();
    }
    auto turned = [&](bool is_k, int h, int i) {
        const float v = turned_plain(is_k, h, i);
        return norm_mode == NORM_UNIT_AFTER ? v * inv[is_k ? H + h : h] : v;
    };
    for (int idx = tid; idx < nq; idx += 256) q_out[static_cast<size_t>(t) * ldq + idx] = from_float<T>(turned(false, idx / d, idx % d));
    if (slot < 0) return;
    T* kp = k_pages + static_cast<size_t>(slot) * nk;
    for (int idx = tid; idx < nk; idx += 256) kp[idx] = from_float<T>(turned(true, idx / d, idx % d));
    T* vp = v_pages + static_cast<size_t>(slot) * G * dv;
    if (v_col < 0) {
        for (int idx = tid; idx < nk; idx += 256) vp[idx] = from_float<T>(ks[idx]);
    } else {
        for (int idx = tid; idx < G * dv; idx += 256) vp[idx] = from_float<T>(row[v_col + idx]);
    }
}

// The same for steps of few rows (decoding), one wavefront per (token, head): queries, then keys. A head of the
// whole-row norm adds up the whole row itself (a few loads a lane) instead of waiting for the other heads. A lane has
// up to 4 columns of its head (d <= 256); rotation partners meet through the wavefront's LDS.
template <typename T>
__global__ void __launch_bounds__(256)
qk_prepare_heads_kernel(const float* __restrict__ proj, int ld, int q_col, int k_col, int v_col, int n_tokens, int H, int G, int d,
                        int dv, int norm_mode, const float* __restrict__ wq, const float* __restrict__ wk, float eps, int rot_dims,
                        double rot_base, int interleaved, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ q_out,
                        int ldq, T* __restrict__ k_pages, T* __restrict__ v_pages) {
    __shared__ float normed_s[4][256];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const int pair = blockIdx.x * 4 + wave;
    if (pair >= n_tokens * (H + G)) return;           // the whole wavefront leaves; no workgroup barrier below
    const int t = pair / (H + G), hh = pair % (H + G);
    const bool is_k = hh >= H;
    const int h = is_k ? hh - H : hh, n_row = (is_k ? G : H) * d;
    const float* row = proj + static_cast<size_t>(t) * ld + (is_k ? k_col : q_col);
    const float* wn = is_k ? wk : wq;
    float raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) raw[u] = row[h * d + min(lane + 64 * u, d - 1)];
    float inv = 1.f;
    if (norm_mode == NORM_HEAD) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) ss += (lane + 64 * u < d) ? raw[u] * raw[u] : 0.f;
        inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(d) + eps);
    } else if (norm_mode == NORM_ROW) {
        float ss = 0.f;
        for (int base = 0; base < n_row; base += 512) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = row[min(base + lane + 64 * u, n_row - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) ss += (base + lane + 64 * u < n_row) ? v[u] * v[u] : 0.f;
        }
        inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(n_row) + eps);
    }
    const int half = rot_dims / 2;
    float* mine = normed_s[threadIdx.x / 64];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = lane + 64 * u;
        if (i < d) {
            float g = 1.f;
            if (norm_mode == NORM_HEAD) g = wn[i];
            if (norm_mode == NORM_ROW) g = wn[h * d + i];
            mine[i] = (norm_mode == NORM_NONE || norm_mode == NORM_UNIT_AFTER) ? raw[u] : raw[u] * inv * g;
        }
    }
    wave_lds_sync();
    const int slot = slots != nullptr ? slots[t] : -1;
    const double pos = static_cast<double>(positions[t]);
    const bool il = interleaved != 0;
    float vals[4];
    float ss_after = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = lane + 64 * u;
        vals[u] = 0.f;
        if (i >= d) continue;
        float val = mine[i];
        if (i < rot_dims) {
            // the angle in double, rounded once
            const int pi = rot_pair(i, half, il);
            const double a = pos * pow(rot_base, -2.0 * pi / rot_dims);
            const float c = static_cast<float>(cos(a)), sn = static_cast<float>(sin(a));
            const float other = mine[rot_partner(i, half, il)];
            val = rot_first(i, half, il) ? val * c - other * sn : val * c + other * sn;
        }
        vals[u] = val;
        ss_after += val * val;
    }
    // (a head scaled to unit root mean square behind the rotation)
    const float inv_after = norm_mode == NORM_UNIT_AFTER ? 1.0f / sqrtf(wave_sum(ss_after) / static_cast<float>(d) + eps) : 1.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = lane + 64 * u;
        if (i >= d) continue;
        const float val = vals[u] * inv_after;
        if (!is_k) q_out[static_cast<size_t>(t) * ldq + h * d + i] = from_float<T>(val);
        else if (slot >= 0) k_pages[static_cast<size_t>(slot) * G * d + h * d + i] = from_float<T>(val);
    }
    if (!is_k || slot < 0) return;
    T* vp = v_pages + static_cast<size_t>(slot) * G * dv + h * dv;
    if (v_col < 0) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (lane + 64 * u < d) vp[lane + 64 * u] = from_float<T>(raw[u]);
    } else {
        const float* vr = proj + static_cast<size_t>(t) * ld + v_col + h * dv;
        for (int i = lane; i < dv; i += 64) vp[i] = from_float<T>(vr[i]);
    }
}

struct ScoreShape {
    float scale, softcap;            // softcap <= 0: none
    int window, chunk;               // at most one of them > 0
    const float* r1;                 // per head, or null: no distance bias
    const float* r2;
    int sigmoid;                     // != 0: a key's weight is sigmoid(score + score_bias[h]), not normalised over the keys
    const float* score_bias;         // per head, or null
    int gate_per_head;               // != 0: the gate has one column per head, not one per value column
    const float* slope;              // per head, or null: s -= slope[h] (i - j)
    const float* sink;               // per head, or null: one more term exp(sink[h]) in the softmax's denominator
    int keep_first;                  // with a window: the first positions that stay visible
};

__device__ __forceinline__ int first_visible(int p, int window, int chunk) {
    if (window > 0) return p - window + 1 > 0 ? p - window + 1 : 0;
    if (chunk > 0) return p - p % chunk;
    return 0;
}

__device__ __forceinline__ float shaped_score(float dot, const ScoreShape& sh, float r1, float r2, int dist) {
    float s = dot * sh.scale;
    if (sh.softcap > 0.f) s = sh.softcap * tanhf(s / sh.softcap);
    if (sh.r1 != nullptr) s -= r1 * log1pf(r2 * static_cast<float>(dist));
    else if (sh.slope != nullptr) s -= r1 * static_cast<float>(dist);        // (r1: the head's slope)
    return s;
}

#define SA_WAVES 4
#define SA_MAX_ACC 8   // value rows of up to 64 * SA_MAX_ACC columns

// One wavefront per (query token, head): 64 keys a round, one key per lane for the scores, then one value
// column (or a few) per lane for the sum. Any sizes; serves prompt portions and single tokens alike.
template <typename T>
__global__ void __launch_bounds__(SA_WAVES * 64)
scored_attention_rows(const T* __restrict__ q, int ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                      const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ token_seq,
                      const int* __restrict__ positions, int n_tokens, int H, int G, int d, int dv, int page_size,
                      ScoreShape sh, const float* __restrict__ gate, int ldg, T* __restrict__ out, int ldo) {
    extern __shared__ float sa_smem[];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int pair = blockIdx.x * SA_WAVES + wave;
    if (pair >= n_tokens * H) return;          // the whole wavefront leaves; no workgroup barrier below
    const int t = pair / H, h = pair % H, hk = h / (H / G);
    const int p = positions[t];
    const int lo = first_visible(p, sh.window, sh.chunk);
    const int* table = block_tables + static_cast<size_t>(token_seq[t]) * max_blocks;
    float* q_s = sa_smem + wave * (d + 128);
    float* p_s = q_s + d;
    int* row_s = reinterpret_cast<int*>(p_s + 64);
    const T* qp = q + static_cast<size_t>(t) * ldq + h * d;
    for (int i = lane; i < d; i += 64) q_s[i] = to_float(qp[i]);
    wave_lds_sync();
    const float r1 = sh.r1 ? sh.r1[h] : (sh.slope ? sh.slope[h] : 0.f), r2 = sh.r1 ? sh.r2[h] : 0.f;
    const float pb = sh.score_bias ? sh.score_bias[h] : 0.f;
    const int kd = G * d, vd = G * dv;
    const bool vec = d % 8 == 0 && (kd * sizeof(T)) % 16 == 0 && (reinterpret_cast<uintptr_t>(k_pages) & 15) == 0;
    float m = -INFINITY, l = 0.f;
    float acc[SA_MAX_ACC];
#pragma unroll
    for (int a = 0; a < SA_MAX_ACC; ++a) acc[a] = 0.f;
    // the visible keys: the window (or chunk, or everything) up to the query, and in front of it the kept first positions
    const int kept_end = (sh.window > 0 && sh.keep_first > 0) ? min(sh.keep_first, lo) : 0;
    for (int seg = kept_end > 0 ? 0 : 1; seg < 2; ++seg) {
    const int seg_end = seg == 0 ? kept_end : p + 1;
    for (int j0 = seg == 0 ? 0 : lo; j0 < seg_end; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < seg_end;
        float s = -INFINITY;
        int row = 0;
        if (valid) {
            row = table[j / page_size] * page_size + j % page_size;
            const T* kp = k_pages + static_cast<size_t>(row) * kd + hk * d;
            float dot = 0.f;
            if (vec) {
                for (int i = 0; i < d; i += 8) {
                    float kv[8];
                    load8(kp + i, kv);
#pragma unroll
                    for (int u = 0; u < 8; ++u) dot = fmaf(q_s[i + u], kv[u], dot);
                }
            } else {
                for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float(kp[i]), dot);
            }
            s = shaped_score(dot, sh, r1, r2, p - j);
        }
        float alpha, pj;
        if (sh.sigmoid) {
            // no softmax: the weight stands for itself, nothing is rescaled or summed
            alpha = 1.f;
            pj = valid ? sigmoid_of(s + pb) : 0.f;
        } else {
            const float m_new = fmaxf(m, wave_max(s));
            alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
            pj = valid ? expf(s - m_new) : 0.f;
            l = l * alpha + wave_sum(pj);
            m = m_new;
        }
        wave_lds_sync();          // the previous round's readers are done
        p_s[lane] = pj;
        row_s[lane] = row;
        wave_lds_sync();
        const int n_keys = min(64, seg_end - j0);
#pragma unroll
        for (int a = 0; a < SA_MAX_ACC; ++a) {
            const int e = lane + a * 64;
            if (e < dv) {
                float o = acc[a] * alpha;
                for (int jj = 0; jj < n_keys; ++jj)
                    o = fmaf(p_s[jj], to_float(v_pages[static_cast<size_t>(row_s[jj]) * vd + hk * dv + e]), o);
                acc[a] = o;
            }
        }
    }
    }
    if (!sh.sigmoid && sh.sink != nullptr) {
        // the sink: a term of the denominator without a value
        const float sk = sh.sink[h], m_new = fmaxf(m, sk);
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * alpha + expf(sk - m_new);
#pragma unroll
        for (int a = 0; a < SA_MAX_ACC; ++a) acc[a] *= alpha;
    }
    T* op = out + static_cast<size_t>(t) * ldo + h * dv;
    const float inv_l = sh.sigmoid ? 1.0f : 1.0f / l;
#pragma unroll
    for (int a = 0; a < SA_MAX_ACC; ++a) {
        const int e = lane + a * 64;
        if (e < dv) {
            float o = acc[a] * inv_l;
            if (gate != nullptr) o *= sigmoid_of(gate[static_cast<size_t>(t) * ldg + (sh.gate_per_head ? h : h * dv + e)]);
            op[e] = from_float<T>(o);
        }
    }
}

// x[t, c] *= sigmoid(gate[t, c])
template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ x, int ldx, const float* __restrict__ gate, int ldg, int N, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / N;
    const int c = static_cast<int>(i % N);
    x[t * ldx + c] = from_float<T>(to_float(x[t * ldx + c]) * sigmoid_of(gate[t * ldg + c]));
}

}  // namespace

extern "C" {

int mllm_gate_mul(void* x, int ldx, const float* gate, int ldg, int T, int N, int dtype, hipStream_t stream) {
    if (T <= 0 || N <= 0) return 0;
    const long long total = static_cast<long long>(T) * N;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32) gate_mul_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<float*>(x), ldx, gate, ldg, N, total);
    else gate_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(x), ldx, gate, ldg, N, total);
    MLLM_LAUNCH_CHECK();
    return 0;
}


// -1: sizes the kernel refuses (an odd rot_dims, rot_dims > d, values from keys with dv != d, more LDS than a
// workgroup has).
int mllm_qk_prepare(const float* proj, int ld, int q_col, int k_col, int v_col, int T, int H, int G, int d, int dv,
                    int norm_mode, const float* wq, const float* wk, float eps, int rot_dims, double rot_base,
                    const int* positions, const int* slots, void* q_out, int ldq, void* k_pages, void* v_pages, int dtype,
                    hipStream_t stream, int interleaved) {
    if (T <= 0) return 0;
    // (G == 0: queries only; the keys and values are another layer's)
    if (H < 1 || G < 0 || d < 1 || dv < 1 || rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > d || rot_dims / 2 > 256) return -1;
    if (v_col < 0 && dv != d) return -1;
    if ((norm_mode == NORM_HEAD || norm_mode == NORM_ROW) && (wq == nullptr || wk == nullptr)) return -1;
    if (norm_mode < NORM_NONE || norm_mode > NORM_UNIT_AFTER) return -1;
    if (T <= 64 && d <= 256) {
        // few rows: one wavefront per (token, head) instead of one workgroup per token
        const int blocks = (T * (H + G) + 3) / 4;
        if (dtype == MLLM_F32)
            qk_prepare_heads_kernel<float><<<blocks, 256, 0, stream>>>(proj, ld, q_col, k_col, v_col, T, H, G, d, dv, norm_mode, wq, wk, eps,
                                                                       rot_dims, rot_base, interleaved, positions, slots, static_cast<float*>(q_out), ldq,
                                                                       static_cast<float*>(k_pages), static_cast<float*>(v_pages));
        else
            qk_prepare_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>(proj, ld, q_col, k_col, v_col, T, H, G, d, dv, norm_mode, wq, wk, eps,
                                                                        rot_dims, rot_base, interleaved, positions, slots, static_cast<bf16_t*>(q_out), ldq,
                                                                        static_cast<bf16_t*>(k_pages), static_cast<bf16_t*>(v_pages));
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const size_t smem = (static_cast<size_t>(H + G) * d + rot_dims + (H + G) + 2) * sizeof(float);
    if (smem > 60 * 1024) return -1;
    if (dtype == MLLM_F32)
        qk_prepare_kernel<float><<<T, 256, smem, stream>>>(proj, ld, q_col, k_col, v_col, H, G, d, dv, norm_mode, wq, wk, eps, rot_dims,
                                                           rot_base, interleaved, positions, slots, static_cast<float*>(q_out), ldq,
                                                           static_cast<float*>(k_pages), static_cast<float*>(v_pages));
    else
        qk_prepare_kernel<bf16_t><<<T, 256, smem, stream>>>(proj, ld, q_col, k_col, v_col, H, G, d, dv, norm_mode, wq, wk, eps, rot_dims,
                                                            rot_base, interleaved, positions, slots, static_cast<bf16_t*>(q_out), ldq,
                                                            static_cast<bf16_t*>(k_pages), static_cast<bf16_t*>(v_pages));
    MLLM_LAUNCH_CHECK();
    return 0;
}

// The keys and values of the step's own tokens must be in the pages. gate (optional): fp32 [T, >= H * dv] with row
// stride ldg (with gate_per_head: [T, >= H]); the result is multiplied by its sigmoid. With sigmoid_weights a key's
// weight is sigmoid(score + score_bias[h]) and there is no softmax. -1: value rows wider than the kernel holds, heads that do
// not group, a window and a chunk at once.
int mllm_scored_attention_rows(const void* q, int ldq, const void* k_pages, const void* v_pages, const int* block_tables,
                               int max_blocks, const int* token_seq, const int* positions, int n_tokens, int H, int G, int d,
                               int dv, int page_size, float scale, float softcap, int window, int chunk, const float* r1,
                               const float* r2, const float* gate, int ldg, void* out, int ldo, int dtype, hipStream_t stream,
                               int sigmoid_weights, const float* score_bias, int gate_per_head, const float* slope,
                               const float* sink, int keep_first) {
    if (n_tokens <= 0) return 0;
    if (H < 1 || G < 1 || H % G != 0 || d < 1 || dv < 1 || dv > 64 * SA_MAX_ACC || page_size < 1) return -1;
    if ((window > 0 && chunk > 0) || window < 0 || chunk < 0 || (r1 != nullptr) != (r2 != nullptr)) return -1;
    const size_t smem = static_cast<size_t>(SA_WAVES) * (d + 128) * sizeof(float);
    if (smem > 60 * 1024) return -1;
    if ((slope != nullptr && r1 != nullptr) || (sink != nullptr && sigmoid_weights) || keep_first < 0) return -1;
    const ScoreShape sh{scale, softcap, window, chunk, r1, r2, sigmoid_weights, score_bias, gate_per_head, slope, sink, keep_first};
    const int blocks = (n_tokens * H + SA_WAVES - 1) / SA_WAVES;
    if (dtype == MLLM_F32)
        scored_attention_rows<float><<<blocks, SA_WAVES * 64, smem, stream>>>(
            static_cast<const float*>(q), ldq, static_cast<const float*>(k_pages), static_cast<const float*>(v_pages), block_tables,
            max_blocks, token_seq, positions, n_tokens, H, G, d, dv, page_size, sh, gate, ldg, static_cast<float*>(out), ldo);
    else
        scored_attention_rows<bf16_t><<<blocks, SA_WAVES * 64, smem, stream>>>(
            static_cast<const bf16_t*>(q), ldq, static_cast<const bf16_t*>(k_pages), static_cast<const bf16_t*>(v_pages), block_tables,
            max_blocks, token_seq, positions, n_tokens, H, G, d, dv, page_size, sh, gate, ldg, static_cast<bf16_t*>(out), ldo);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
