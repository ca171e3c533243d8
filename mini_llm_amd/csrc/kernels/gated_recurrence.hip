// Linear recurrences with a decay per key channel, for gfx950. Per head with d key channels and dv value
// channels, token by token:
//   S[i, e] <- f_i S[i, e] + k_i v_e;   o_e = sum_i S[i, e] q_i
// in two forms. FORM 0, a forget gate that also decides what is written (HGRN2):
//   f_i = l_i + (1 - l_i) sigmoid(fraw_i + b_i)  (a lower bound l per channel),  k_i = 1 - f_i,  q_i = silu(qraw_i)
// FORM 1, keys of their own (linear attention with a decay): q_i = q_scale * qraw_i, k_i = k_scale * kraw_i, and
// f_i either read per token and channel from an array of decays or one constant per head.
// The state S ([head][d][dv], dv contiguous, fp32) lives in a per-request slot and is carried from step to
// step. Gates, state and sums are fp32; the inputs are the fp32 rows of the input projection.
//
// One wavefront per (sequence, head, 64 value columns, slice of GR_ROWS key channels): a lane owns one value
// column and keeps its slice of the state in registers; the gate and the query of a slice's channel are the
// same for all lanes, so lane i works them out for channel i and they go round through LDS. The sum over the
// key channels is split over the slices: slice s leaves its share in y + s * part_stride, and the reader (the
// norm that follows) adds the shares in the order of s.
#include "common.h"

#define GR_ROWS 32

namespace {

__device__ __forceinline__ float gr_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }

// MODE 0: every portion of the step is one chunk: from the slot's state, results to y, the state back to the slot.
// Portions longer than GR_CHUNK tokens are cut into chunks that run side by side, in three launches:
// MODE 1: every chunk from a zero state; it leaves its last state and the product of its gates in the workspace;
//         then hgrn2_chunk_states_kernel walks a sequence's chunks in order, S <- F_c S + L_c, leaves in the
//         workspace the state each chunk starts from, and writes the last state to the slot;
// MODE 2: every chunk again, from the state it starts from, results to y.
// The sums are those of the token-by-token recurrence in another order.
// Workspace per chunk and head: [d * dv] the chunk's state, then [d] the product of its gates.
#define GR_CHUNK 32

// What FORM 1 reads besides the projection's rows: the decays per token and channel ([T, ldd] fp32, heads * d
// columns), or, if that is null, one decay per head; and the two scales.
struct KeyedDecay {
    const float* decay;
    int ldd;
    const float* head_decay;
    float q_scale, k_scale;
};

template <int MODE, int FORM>
__global__ void __launch_bounds__(64)
hgrn2_scan_kernel(const float* __restrict__ proj, int ld, int q_col, int f_col, int v_col, const float* __restrict__ f_bias,
                  const float* __restrict__ lower, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                  float* __restrict__ state, size_t slot_floats, float* __restrict__ y, int ldy, size_t part_stride, int H, int d,
                  int dv, int n_tiles, int n_slices, int write, int n_seqs, float* __restrict__ ws, KeyedDecay kd) {
    // per token in turn: [f | q] of the slice's channels, and in FORM 1 [k] behind them (f_col is then the keys' column)
    __shared__ float fq[2][3 * GR_ROWS];
    const int lane = threadIdx.x;
    int w = blockIdx.x;
    const int slice = w % n_slices; w /= n_slices;
    const int tile = w % n_tiles; w /= n_tiles;
    const int h = w % H;
    w /= H;
    int b, first, n, chunk_id = 0;
    if (MODE == 0) {
        b = w;
        first = cu_q[b];
        n = cu_q[b + 1] - first;
    } else {
        // which sequence and which of its chunks
        chunk_id = w;
        int c = w;
        for (b = 0; b < n_seqs; ++b) {
            first = cu_q[b];
            n = cu_q[b + 1] - first;
            const int nc = (n + GR_CHUNK - 1) / GR_CHUNK;
            if (c < nc) break;
            c -= nc;
        }
        if (b >= n_seqs) return;                // a surplus workgroup
        first += c * GR_CHUNK;
        n = min(GR_CHUNK, n - c * GR_CHUNK);
    }
    const int slot = state_slots[b];
    if (slot < 0) return;
    const int e = tile * 64 + lane, i0 = slice * GR_ROWS;
    const int rows = min(GR_ROWS, d - i0);
    const bool col_ok = e < dv;
    float* S = state + static_cast<size_t>(slot) * slot_floats + (static_cast<size_t>(h) * d + i0) * dv + (col_ok ? e : 0);
    float* W = ws ? ws + (static_cast<size_t>(chunk_id) * H + h) * (static_cast<size_t>(d) * dv + d) : nullptr;
    float* WS = W ? W + static_cast<size_t>(i0) * dv + (col_ok ? e : 0) : nullptr;
    float s[GR_ROWS];
#pragma unroll
    for (int i = 0; i < GR_ROWS; ++i) {
        // (the start: the slot's state, zero, or what the pass over the chunks left for this chunk)
        const float* from = MODE == 2 ? WS : S;
        s[i] = (MODE != 1 && i < rows && col_ok) ? from[static_cast<size_t>(i) * dv] : 0.f;
    }
    // the channel this lane prepares: lanes 0..31 the gate of channel lane, lanes 32..63 the query of channel lane - 32
    const int ch = lane % GR_ROWS;
    const bool ch_ok = ch < rows;
    const int c = h * d + i0 + (ch_ok ? ch : 0);
    const float lo = FORM == 0 ? lower[c] : 0.f, fb = (FORM == 0 && f_bias) ? f_bias[c] : 0.f;
    float cum = 1.f;                            // (lanes 0..31) the product of the channel's gates over the chunk
    // A token's inputs are asked for one token ahead (from a clamped, always valid row), so that the round trip to
    // memory runs beside the arithmetic of the token before.
    const int col = lane < GR_ROWS ? f_col + c : q_col + c;
    const int vcol = v_col + h * dv + (col_ok ? e : 0);
    const bool per_token = FORM == 1 && kd.decay != nullptr;
    const float fixed = (FORM == 1 && !per_token) ? kd.head_decay[h] : 0.f;
    float raw = 0.f, v_next = 0.f, dec_next = fixed;
    if (n > 0) {
        raw = proj[static_cast<size_t>(first) * ld + col];
        v_next = proj[static_cast<size_t>(first) * ld + vcol];
        if (per_token) dec_next = kd.decay[static_cast<size_t>(first) * kd.ldd + c];
    }
    for (int k = 0; k < n; ++k) {
        const float z = raw, v = col_ok ? v_next : 0.f, dec = dec_next;
        const size_t row_ahead = static_cast<size_t>(first + min(k + 1, n - 1));
        const float* ahead = proj + row_ahead * ld;
        raw = ahead[col];
        v_next = ahead[vcol];
        if (per_token) dec_next = kd.decay[row_ahead * kd.ldd + c];
        float* cur = fq[k & 1];
        if (FORM == 0) {
            float val;
            if (lane < GR_ROWS) { val = lo + (1.f - lo) * gr_sigmoid(z + fb); cum *= val; }
            else val = z * gr_sigmoid(z);
            cur[lane] = ch_ok ? val : 0.f;
        } else {
            // lanes 0..31: the channel's decay and its key; lanes 32..63: its query
            if (lane < GR_ROWS) {
                cum *= dec;
                cur[lane] = ch_ok ? dec : 0.f;
                cur[2 * GR_ROWS + lane] = ch_ok ? z * kd.k_scale : 0.f;
            } else {
                cur[lane] = ch_ok ? z * kd.q_scale : 0.f;
            }
        }
        wave_lds_sync();
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < GR_ROWS; ++i) {
            const float f = cur[i], qi = cur[GR_ROWS + i];
            if (FORM == 0) s[i] = f * s[i] + (1.f - f) * v;
            else s[i] = fmaf(f, s[i], cur[2 * GR_ROWS + i] * v);
            o = fmaf(s[i], qi, o);
        }
        if (MODE != 1 && col_ok) y[slice * part_stride + static_cast<size_t>(first + k) * ldy + h * dv + e] = o;
    }
    if (MODE == 0 && write && col_ok) {
#pragma unroll
        for (int i = 0; i < GR_ROWS; ++i)
            if (i < rows) S[static_cast<size_t>(i) * dv] = s[i];
    }
    if (MODE == 1) {
        if (col_ok) {
#pragma unroll
            for (int i = 0; i < GR_ROWS; ++i)
                if (i < rows) WS[static_cast<size_t>(i) * dv] = s[i];
        }
        if (tile == 0 && lane < GR_ROWS && ch_ok) W[static_cast<size_t>(d) * dv + i0 + ch] = cum;
    }
}

// One thread per (sequence, head, key channel, value column): the sequence's chunks in order. In the workspace a
// chunk's own last state is replaced by the state it starts from.
__global__ void hgrn2_chunk_states_kernel(const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ state,
                                          size_t slot_floats, float* __restrict__ ws, int H, int d, int dv, int n_seqs, int write) {
    const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const long long per_seq = static_cast<long long>(H) * d * dv;
    if (idx >= per_seq * n_seqs) return;
    const int b = static_cast<int>(idx / per_seq);
    const long long r = idx % per_seq;
    const int h = static_cast<int>(r / (static_cast<long long>(d) * dv)), i = static_cast<int>(r / dv % d);
    const int slot = state_slots[b];
    if (slot < 0) return;
    int chunk0 = 0;
    for (int bb = 0; bb < b; ++bb) chunk0 += (cu_q[bb + 1] - cu_q[bb] + GR_CHUNK - 1) / GR_CHUNK;
    const int nc = (cu_q[b + 1] - cu_q[b] + GR_CHUNK - 1) / GR_CHUNK;
    float* sp = state + static_cast<size_t>(slot) * slot_floats + r;
    float S = *sp;
    const size_t per_chunk = static_cast<size_t>(d) * dv + d;
    for (int c = 0; c < nc; ++c) {
        float* W = ws + (static_cast<size_t>(chunk0 + c) * H + h) * per_chunk;
        const float L = W[r % (static_cast<long long>(d) * dv)], F = W[static_cast<size_t>(d) * dv + i];
        W[r % (static_cast<long long>(d) * dv)] = S;
        S = F * S + L;
    }
    if (write) *sp = S;
}

// out[t, :] = [a[t, :] | b[t, :]] in the output's dtype (two fp32 streams side by side, as one product's input)
template <typename T>
__global__ void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b, int D, T* __restrict__ out, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / (2 * D);
    const int c = static_cast<int>(i % (2 * D));
    out[i] = from_float<T>(c < D ? a[t * D + c] : b[t * D + c - D]);
}

// out[t, j] = act(gu[t, j]) * gu[t, F + j]: the two halves of a joined gate/up product
template <typename T, bool SILU>
__global__ void glu_act_kernel(const T* __restrict__ gu, int ld, int F, T* __restrict__ out, int ldo, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / F;
    const int j = static_cast<int>(i % F);
    const float g = to_float(gu[t * ld + j]), u = to_float(gu[t * ld + F + j]);
    if (SILU) out[t * ldo + j] = from_float<T>(g / (1.f + (sizeof(T) == 4 ? expf(-g) : __expf(-g))) * u);
    else out[t * ldo + j] = from_float<T>((sizeof(T) == 4 ? gelu_tanh_precise(g) : gelu_tanh(g)) * u);
}


// proj[t, col0 + hh * d + i] for hh < n_heads, i < rot_dims, turned in place by the token's position: column i pairs
// with i + rot_dims / 2, the pair (a, b) becomes (a cos - b sin, b cos + a sin) of the angle p * base^(-2i / rot_dims)
// (worked out in double, rounded once). One thread per pair.
__global__ void rotary_rows_kernel(float* __restrict__ proj, int ld, int col0, int n_heads, int d, int rot_dims, double base,
                                   const int* __restrict__ positions, long long total) {
    const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int half = rot_dims / 2;
    const int i = static_cast<int>(idx % half);
    const int hh = static_cast<int>(idx / half % n_heads);
    const long long t = idx / (static_cast<long long>(half) * n_heads);
    const double a = static_cast<double>(positions[t]) * pow(base, -2.0 * i / rot_dims);
    const float c = static_cast<float>(cos(a)), sn = static_cast<float>(sin(a));
    float* p = proj + static_cast<size_t>(t) * ld + col0 + hh * d + i;
    const float u = p[0], v = p[half];
    p[0] = u * c - v * sn;
    p[half] = v * c + u * sn;
}

// out[t, c] = sigmoid(z)^(1 / tau) with z = bias[c] + sum_r w[c, r] * proj[t, a_col + r]: the decays of a recurrence from
// a low-rank map of the input whose first half (rank values per token) the input projection has already made.
// exp(log sigmoid(z) / tau) with log sigmoid(z) = min(z, 0) - log1p(exp(-|z|)). One thread per (token, channel);
// the token's rank values go through LDS.
__global__ void __launch_bounds__(256)
lowrank_decay_kernel(const float* __restrict__ proj, int ld, int a_col, int rank, const float* __restrict__ w, const float* __restrict__ bias,
                     float inv_tau, float* __restrict__ out, int ldo, int N) {
    extern __shared__ float lr_smem[];
    const int t = blockIdx.y;
    for (int r = threadIdx.x; r < rank; r += 256) lr_smem[r] = proj[static_cast<size_t>(t) * ld + a_col + r];
    __syncthreads();
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= N) return;
    float z = bias ? bias[c] : 0.f;
    const float* wr = w + static_cast<size_t>(c) * rank;
    for (int r = 0; r < rank; ++r) z = fmaf(wr[r], lr_smem[r], z);
    const float ls = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
    out[static_cast<size_t>(t) * ldo + c] = expf(ls * inv_tau);
}

}  // namespace

namespace {
template <int FORM>
int launch_scan(const float* proj, int ld, int q_col, int f_col, int v_col, const float* f_bias, const float* lower, const int* cu_q,
                const int* state_slots, float* state, size_t slot_floats, size_t state_offset, float* y, int ldy, size_t part_stride, int T,
                int B, int max_q_len, int H, int d, int dv, int write, float* workspace, const KeyedDecay& kd, hipStream_t stream) {
    const int n_tiles = (dv + 63) / 64, n_slices = (d + GR_ROWS - 1) / GR_ROWS;
    const long long per = static_cast<long long>(H) * n_tiles * n_slices;
    if (max_q_len <= GR_CHUNK || workspace == nullptr) {
        if (per * B >= (1ll << 31)) return -1;
        hgrn2_scan_kernel<0, FORM><<<static_cast<int>(per * B), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                                state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                                n_tiles, n_slices, write, B, nullptr, kd);
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const long long chunks = T / GR_CHUNK + B;          // an upper bound; surplus workgroups leave at once
    if (per * chunks >= (1ll << 31)) return -1;
    hgrn2_scan_kernel<1, FORM><<<static_cast<int>(per * chunks), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                                 state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                                 n_tiles, n_slices, write, B, workspace, kd);
    MLLM_LAUNCH_CHECK();
    const long long cells = static_cast<long long>(B) * H * d * dv;
    hgrn2_chunk_states_kernel<<<static_cast<int>((cells + 255) / 256), 256, 0, stream>>>(cu_q, state_slots, state + state_offset, slot_floats,
                                                                                        workspace, H, d, dv, B, write);
    MLLM_LAUNCH_CHECK();
    hgrn2_scan_kernel<2, FORM><<<static_cast<int>(per * chunks), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                                 state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                                 n_tiles, n_slices, write, B, workspace, kd);
    MLLM_LAUNCH_CHECK();
    return 0;
}
}  // namespace

extern "C" {

int mllm_hgrn2_parts(int d) { return (d + GR_ROWS - 1) / GR_ROWS; }

// proj [T, ld] fp32 holds, per token, the raw queries (H * d from q_col), raw gates (H * d from f_col) and values
// (H * dv from v_col). y: mllm_hgrn2_parts(d) shares of [T, ldy], part_stride floats apart. The state of a
// request lies state_offset floats into its slot.
int mllm_hgrn2_scan(const float* proj, int ld, int q_col, int f_col, int v_col, const float* f_bias, const float* lower,
                    const int* cu_q, const int* state_slots, float* state, size_t slot_floats, size_t state_offset, float* y, int ldy,
                    size_t part_stride, int T, int B, int max_q_len, int H, int d, int dv, int write, float* workspace,
                    hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (H < 1 || d < 1 || dv < 1 || lower == nullptr) return -1;
    return launch_scan<0>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots, state, slot_floats, state_offset, y, ldy, part_stride, T,
                          B, max_q_len, H, d, dv, write, workspace, KeyedDecay{nullptr, 0, nullptr, 1.f, 1.f}, stream);
}

// The recurrence with keys of its own: queries (H * d from q_col), keys (H * d from k_col) and values (H * dv from
// v_col) in proj's fp32 rows; the decays per token and channel in `decay` ([T, ldd] fp32, H * d columns), or, if that
// is null, one per head in `head_decay` ([H]). Shares, state and workspace as for mllm_hgrn2_scan.
int mllm_decay_scan(const float* proj, int ld, int q_col, int k_col, int v_col, const float* decay, int ldd, const float* head_decay,
                    float q_scale, float k_scale, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                    size_t state_offset, float* y, int ldy, size_t part_stride, int T, int B, int max_q_len, int H, int d, int dv, int write,
                    float* workspace, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (H < 1 || d < 1 || dv < 1 || (decay == nullptr && head_decay == nullptr)) return -1;
    return launch_scan<1>(proj, ld, q_col, k_col, v_col, nullptr, nullptr, cu_q, state_slots, state, slot_floats, state_offset, y, ldy, part_stride,
                          T, B, max_q_len, H, d, dv, write, workspace, KeyedDecay{decay, ldd, head_decay, q_scale, k_scale}, stream);
}

// Turns the first rot_dims columns of n_heads heads of d columns, from column col0 of proj's fp32 rows, in place.
// -1: an odd rot_dims or one beyond the head.
int mllm_rotary_rows(float* proj, int ld, int col0, int T, int n_heads, int d, int rot_dims, double base, const int* positions,
                     hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || rot_dims == 0) return 0;
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > d || !(base > 0)) return -1;
    const long long total = static_cast<long long>(T) * n_heads * (rot_dims / 2);
    rotary_rows_kernel<<<static_cast<int>((total + 255) / 256), 256, 0, stream>>>(proj, ld, col0, n_heads, d, rot_dims, base, positions, total);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// out [T, N] fp32 = sigmoid(w proj[:, a_col : a_col + rank] + bias)^(1 / tau); w [N, rank] fp32. -1: a rank beyond 8,192
// or a tau that is not positive.
int mllm_lowrank_decay(const float* proj, int ld, int a_col, int rank, const float* w, const float* bias, float tau, float* out, int ldo,
                       int T, int N, hipStream_t stream) {
    if (T <= 0 || N <= 0) return 0;
    if (rank < 1 || rank > 8192 || !(tau > 0.f) || T > 65535 * 32) return -1;
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int n = T - t0 < 65535 ? T - t0 : 65535;
        lowrank_decay_kernel<<<dim3((N + 255) / 256, n), 256, rank * sizeof(float), stream>>>(proj + static_cast<size_t>(t0) * ld, ld, a_col, rank, w,
                                                                                             bias, 1.0f / tau, out + static_cast<size_t>(t0) * ldo, ldo, N);
    }
    MLLM_LAUNCH_CHECK();
    return 0;
}

// Floats of workspace that a step of T tokens in B sequences needs when its longest portion exceeds a chunk.
size_t mllm_hgrn2_workspace_floats(int T, int B, int H, int d, int dv) {
    return static_cast<size_t>(T / GR_CHUNK + B) * H * (static_cast<size_t>(d) * dv + d);
}
int mllm_hgrn2_chunk() { return GR_CHUNK; }

int mllm_concat_cast(const float* a, const float* b, int T, int D, void* out, int dtype, hipStream_t stream) {
    if (T <= 0 || D <= 0) return 0;
    const long long total = static_cast<long long>(T) * 2 * D;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32) concat_cast_kernel<float><<<blocks, 256, 0, stream>>>(a, b, D, static_cast<float*>(out), total);
    else concat_cast_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, b, D, static_cast<bf16_t*>(out), total);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// -1: an activation other than the tanh form of GELU (code 1) or silu (code 5)
int mllm_glu_act(const void* gu, int ld, int T, int F, int act, void* out, int ldo, int dtype, hipStream_t stream) {
    if (T <= 0 || F <= 0) return 0;
    if (act != EPI_GELU_TANH && act != 5) return -1;
    const long long total = static_cast<long long>(T) * F;
    const int blocks = static_cast<int>((total + 255) / 256);
#define GLU_ACT(TYPE, SILU) glu_act_kernel<TYPE, SILU><<<blocks, 256, 0, stream>>>(static_cast<const TYPE*>(gu), ld, F, static_cast<TYPE*>(out), ldo, total)
    if (dtype == MLLM_F32) { if (act == 5) GLU_ACT(float, true); else GLU_ACT(float, false); }
    else { if (act == 5) GLU_ACT(bf16_t, true); else GLU_ACT(bf16_t, false); }
#undef GLU_ACT
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
