// State-space mixer kernels for gfx950: the short causal convolution with its carried inputs, and the
// selective scan (Mamba-2 form: one decay per head and token) over a step's portions, the state carried
// in a per-request slot. Everything here is fp32.
//
// A request's slot holds [taps - 1][channels] convolution inputs (oldest first), then the scan's state
// laid out [head][n][p] (p contiguous).
#include <algorithm>

#include "common.h"

namespace {

__device__ __forceinline__ float silu_precise(float v) { return v / (1.f + expf(-v)); }
// log(1 + exp(v)) without overflow, no clamp
__device__ __forceinline__ float softplus_precise(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// out[t, ch] = silu(bias[ch] + sum_j w[ch, j] * in(t - (taps - 1 - j), ch)): inputs before the portion come
// from the slot's carried rows (zeros for a fresh request: the slot was cleared). One thread per (t, ch).
__global__ void conv_silu_kernel(const float* __restrict__ proj, int ld, int col0, int C, const float* __restrict__ w,
                                 const float* __restrict__ bias, int taps, const int* __restrict__ token_seq,
                                 const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                 float* __restrict__ state, size_t slot_floats, float* __restrict__ out, int ldo,
                                 long long total, int carry) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / C), ch = static_cast<int>(i % C);
    const int b = token_seq[t], slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], k = t - first;
    float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float acc = bias[ch];
    for (int j = 0; j < taps; ++j) {
        const int idx = k - (taps - 1 - j);
        const float v = idx >= 0 ? proj[static_cast<size_t>(first + idx) * ld + col0 + ch]
                                 : carried[static_cast<size_t>(taps - 1 + idx) * C + ch];
        acc += w[static_cast<size_t>(ch) * taps + j] * v;
        // `carry` (every portion of the step is a single token, so this thread is the channel's only reader): the
        // carried rows move up by one behind the read, and the token's input becomes the newest
        if (carry && j >= 1) carried[static_cast<size_t>(j - 1) * C + ch] = v;
    }
    out[static_cast<size_t>(t) * ldo + ch] = silu_precise(acc);
}

// out[t, ch] = in[t, ch] + sum_j w[ch, j] * in(t - (taps - 1 - j), ch): the convolution added onto its own input,
// no bias and no activation, the result in the activation dtype. Carried rows as above. residual == 0: the
// convolution alone, its input not added.
template <typename OutT>
__global__ void conv_residual_kernel(const float* __restrict__ in, int ld, int C, const float* __restrict__ w, int taps,
                                     const int* __restrict__ token_seq, const int* __restrict__ cu_q,
                                     const int* __restrict__ state_slots, float* __restrict__ state, size_t slot_floats,
                                     OutT* __restrict__ out, int ldo, long long total, int carry, int residual) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / C), ch = static_cast<int>(i % C);
    const int b = token_seq[t], slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], k = t - first;
    float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float acc = 0.f, own = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int idx = k - (taps - 1 - j);
        const float v = idx >= 0 ? in[static_cast<size_t>(first + idx) * ld + ch]
                                 : carried[static_cast<size_t>(taps - 1 + idx) * C + ch];
        acc += w[static_cast<size_t>(ch) * taps + j] * v;
        own = v;
        if (carry && j >= 1) carried[static_cast<size_t>(j - 1) * C + ch] = v;
    }
    out[static_cast<size_t>(t) * ldo + ch] = from_float<OutT>(residual ? own + acc : acc);
}

// The same four channels a thread (16-byte loads; the rows' widths and the places are multiples of four floats). A
// token with taps - 1 tokens of its own portion in front of it reads them all from `in`, without conditions, so its
// loads are in flight together; the first tokens of a portion read the slot's carried rows where the portion has none.
// A wavefront holds one token's channels (or the border of two tokens), so the two ways seldom meet in one.
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}
template <typename OutT, int TAPS>
__global__ void conv_residual_vec_kernel(const float* __restrict__ in, int ld, int C, const float* __restrict__ w,
                                         const int* __restrict__ token_seq, const int* __restrict__ cu_q,
                                         const int* __restrict__ state_slots, float* __restrict__ state, size_t slot_floats,
                                         OutT* __restrict__ out, int ldo, long long total4, int carry, int residual) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total4) return;
    const int C4 = C / 4;
    const int t = static_cast<int>(i / C4), ch = static_cast<int>(i % C4) * 4;
    const int b = token_seq[t], slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], k = t - first;
    float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float4 wf[TAPS], v[TAPS];             // wf: the four channels' taps one behind the other (4 * TAPS floats)
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wf[j] = *reinterpret_cast<const float4*>(w + static_cast<size_t>(ch) * TAPS + 4 * j);
    if (k >= TAPS - 1) {
#pragma unroll
        for (int j = 0; j < TAPS; ++j) v[j] = *reinterpret_cast<const float4*>(in + static_cast<size_t>(t - (TAPS - 1 - j)) * ld + ch);
    } else {
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            const int idx = k - (TAPS - 1 - j);
            v[j] = idx >= 0 ? *reinterpret_cast<const float4*>(in + static_cast<size_t>(first + idx) * ld + ch)
                            : *reinterpret_cast<const float4*>(carried + static_cast<size_t>(TAPS - 1 + idx) * C + ch);
        }
    }
    float wv[4 * TAPS];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) { wv[4 * j] = wf[j].x; wv[4 * j + 1] = wf[j].y; wv[4 * j + 2] = wf[j].z; wv[4 * j + 3] = wf[j].w; }
    float r[4] = {v[TAPS - 1].x, v[TAPS - 1].y, v[TAPS - 1].z, v[TAPS - 1].w};
    if (!residual) r[0] = r[1] = r[2] = r[3] = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
        acc[0] += wv[0 * TAPS + j] * v[j].x;
        acc[1] += wv[1 * TAPS + j] * v[j].y;
        acc[2] += wv[2 * TAPS + j] * v[j].z;
        acc[3] += wv[3 * TAPS + j] * v[j].w;
    }
    if (carry) {
#pragma unroll
        for (int j = 1; j < TAPS; ++j) *reinterpret_cast<float4*>(carried + static_cast<size_t>(j - 1) * C + ch) = v[j];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) r[q] += acc[q];
    store4(out + static_cast<size_t>(t) * ldo + ch, r);
}

// A step in which every sequence brings one token: h = x / sqrt(mean(x^2) + eps) * wn and out = h + conv(h) in one
// kernel, one workgroup per token. The earlier inputs of the convolution are the slot's carried rows, which move up
// by one behind the read; h becomes the newest.
// NB wavefronts, each with a block of 512 columns: its part of the row stays in registers between the statistics (the
// wavefronts' sums meet in LDS and are added in the order of the blocks) and the convolution. All loads of a block
// are issued together, without conditions, from clamped (always valid) places, and masked where they are used (a
// load under a condition, or in a loop of unknown length, is waited for before the next is asked for); TAPS is a
// constant for that reason.
// MODE 0: as above. MODE 1, a norm BEHIND a sub-layer and the next sub-layer's convolution: the stream's row becomes
// x + y / sqrt(mean(y^2) + eps) * wn (y: the sub-layer's result; x is written back), and h is that row. MODE 2: no norm,
// h = x.
template <typename OutT, int TAPS, int NB, int MODE>
__global__ void __launch_bounds__(64 * NB)
rmsnorm_conv_single_kernel(float* x, int ldx, const float* __restrict__ y, int ldy, const float* __restrict__ wn, float eps, int C,
                           const float* __restrict__ wc, const int* __restrict__ state_slots, float* __restrict__ state,
                           size_t slot_floats, OutT* __restrict__ out, int ldo, int write) {
    __shared__ float part[NB];
    const int b = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int t = blockIdx.x;
    const int slot = state_slots[t];
    if (slot < 0) return;                      // (the whole workgroup: one token)
    float* xr = x + static_cast<size_t>(t) * ldx;
    int idx[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) idx[u] = min(512 * b + lane + 64 * u, C - 1);
    float xv[8], yv[8], g[8], w[TAPS][8], v[TAPS > 1 ? TAPS - 1 : 1][8];
#pragma unroll
    for (int u = 0; u < 8; ++u) xv[u] = xr[idx[u]];
    if (MODE == 1) {
        const float* yr = y + static_cast<size_t>(t) * ldy;
#pragma unroll
        for (int u = 0; u < 8; ++u) yv[u] = yr[idx[u]];
    }
    const float* carried = state + static_cast<size_t>(slot) * slot_floats;
#pragma unroll
    for (int u = 0; u < 8; ++u) g[u] = MODE == 2 ? 1.f : wn[idx[u]];
#pragma unroll
    for (int j = 0; j < TAPS; ++j)
#pragma unroll
        for (int u = 0; u < 8; ++u) w[j][u] = wc[static_cast<size_t>(idx[u]) * TAPS + j];
#pragma unroll
    for (int j = 0; j + 1 < TAPS; ++j)
#pragma unroll
        for (int u = 0; u < 8; ++u) v[j][u] = carried[static_cast<size_t>(j) * C + idx[u]];
    float inv = 1.f;
    if (MODE != 2) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float z = MODE == 1 ? yv[u] : xv[u];
            ss += (512 * b + lane + 64 * u < C) ? z * z : 0.f;
        }
        ss = wave_sum(ss);
        if (NB > 1) {
            if (lane == 0) part[b] = ss;
            __syncthreads();
            ss = 0.f;
#pragma unroll
            for (int k = 0; k < NB; ++k) ss += part[k];
        }
        inv = 1.0f / sqrtf(ss / static_cast<float>(C) + eps);
    }
    float* carried_w = state + static_cast<size_t>(slot) * slot_floats;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const float h = MODE == 0 ? xv[u] * inv * g[u] : MODE == 1 ? xv[u] + yv[u] * inv * g[u] : xv[u];
        float acc = w[TAPS - 1][u] * h;
#pragma unroll
        for (int j = 0; j + 1 < TAPS; ++j) acc += w[j][u] * v[j][u];
        if (512 * b + lane + 64 * u < C) {
            if (MODE == 1) xr[idx[u]] = h;
            if (write) {
#pragma unroll
                for (int j = 1; j + 1 < TAPS; ++j) carried_w[static_cast<size_t>(j - 1) * C + idx[u]] = v[j][u];
                if (TAPS > 1) carried_w[static_cast<size_t>(TAPS - 2) * C + idx[u]] = h;
            }
            out[static_cast<size_t>(t) * ldo + idx[u]] = from_float<OutT>(h + acc);
        }
    }
}

// The slot's carried rows after the portion: its last taps - 1 inputs, older ones shifted out; a portion
// shorter than that keeps the newest of the old rows. One thread per (sequence, channel); taps - 1 <= 15.
__global__ void conv_carry_kernel(const float* __restrict__ proj, int ld, int col0, int C, int taps,
                                  const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                  float* __restrict__ state, size_t slot_floats, int B) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= static_cast<long long>(B) * C) return;
    const int b = static_cast<int>(i / C), ch = static_cast<int>(i % C);
    const int slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], n = cu_q[b + 1] - first, keep = taps - 1;
    float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float fresh[15];
#pragma unroll
    for (int r = 0; r < 15; ++r) {
        if (r < keep) {
            const int idx = n - keep + r;
            fresh[r] = idx >= 0 ? proj[static_cast<size_t>(first + idx) * ld + col0 + ch]
                                : carried[static_cast<size_t>(r + n) * C + ch];
        }
    }
#pragma unroll
    for (int r = 0; r < 15; ++r)
        if (r < keep) carried[static_cast<size_t>(r) * C + ch] = fresh[r];
}

// The scan. For head h (group g = h / (H / G)) and token t, in order:
//   dt = softplus(raw_dt[t, h] + dt_bias[h]);  a = exp(-exp(A_log[h]) dt)
//   S[n, p] = a S[n, p] + dt B[t, g, n] x[t, h, p];   y[t, h, p] = sum_n S[n, p] C[t, g, n] + D[h] x[t, h, p]
// One wavefront per (chunk of a sequence's portion, head, 64 values of p, slice of NS values of n): a lane owns
// one p and keeps its NS state values in registers, so B and C of the slice are the same for the whole wavefront
// (they arrive as scalars) and x is one coalesced load. The sum over n is split over the slices: slice s leaves its
// share in y + s * part_stride, and the reader (the gated norm) adds the shares in the order of s. The state in a
// slot is laid out [head][n][p] (p contiguous). xbc rows: [x: H*P | B: G*N | C: G*N].
//
// A portion longer than `chunk` tokens is cut into chunks that are scanned side by side: the first starts
// from the slot's state, the others from zero, and each leaves its last state in `chunk_state`
// ([chunk][H][N][P]) and, per token, the logarithm of the decay accumulated since its chunk began in `cumlog`
// ([T, H]). ssm_chunk_join_kernel then adds what the earlier chunks contribute. A portion of one chunk
// (decoding) is finished here and its state goes straight back to the slot.
struct ChunkOf {
    int b, k, n_chunks, first_chunk;      // sequence, chunk within it, chunks of the sequence, where its chunks' states start
                                          // (only portions of several chunks keep states: at most 2 T / chunk of them)
};
__device__ __forceinline__ ChunkOf chunk_of(int index, const int* cu_q, int n_seqs, int chunk, bool chunked) {
    // (no portion longer than a chunk: chunk i is sequence i, and no walk over the sequences, whose every step
    // would wait for a load)
    if (!chunked) return ChunkOf{index < n_seqs ? index : -1, 0, 1, 0};
    ChunkOf c{0, index, 0, 0};
    for (; c.b < n_seqs; ++c.b) {
        c.n_chunks = max(1, (cu_q[c.b + 1] - cu_q[c.b] + chunk - 1) / chunk);
        if (c.k < c.n_chunks) return c;
        c.k -= c.n_chunks;
        if (c.n_chunks > 1) c.first_chunk += c.n_chunks;
    }
    c.b = -1;
    return c;
}

template <int NS>
__global__ void __launch_bounds__(64)
ssm_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ raw_dt, int ldd,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
                const int* __restrict__ cu_q, const int* __restrict__ state_slots, int n_seqs, float* __restrict__ state,
                size_t slot_floats, size_t scan_offset, float* __restrict__ y, int ldy, size_t part_stride, int H, int P,
                int N, int G, int n_slices, int write, int chunk, float* __restrict__ chunk_state,
                float* __restrict__ cumlog) {
    const int lane = threadIdx.x;
    const int h = blockIdx.y, slice = blockIdx.x % n_slices, p = (blockIdx.x / n_slices) * 64 + lane;
    const ChunkOf co = chunk_of(blockIdx.z, cu_q, n_seqs, chunk, chunk_state != nullptr);
    if (co.b < 0) return;                                      // surplus workgroup
    const int slot = state_slots[co.b];
    if (slot < 0) return;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int n0 = slice * NS, nn = min(NS, N - n0);
    const int t0 = cu_q[co.b] + co.k * chunk, t1 = min(t0 + chunk, cu_q[co.b + 1]);
    float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * N + n0) * P + pc;
    // (every load below is issued without a condition, from a clamped index, and masked by a select afterwards: a
    // load under a condition waits for all loads in flight, which would make a token cost NS round trips)
    float S[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = sp[static_cast<size_t>(min(j, nn - 1)) * P];
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = (co.k == 0 && j < nn) ? S[j] : 0.f;
    const float bias = dt_bias[h], neg_rate = -expf(A_log[h]), skip = slice == 0 ? Dskip[h] : 0.f;
    const float* b_row = xbc + inner + g * N + n0;              // + t * ldx: B of the slice (the same for every lane)
    const float* c_row = b_row + G * N;
    float* yp = y + slice * part_stride + h * P + pc;
    // a token's operands are requested one token ahead; rows of the slice beyond N count as zeros
    float xv = 0.f, dtr = 0.f, Bv[NS], Cv[NS];
    auto load = [&](int t, float& x_, float& d_, float (&B_)[NS], float (&C_)[NS]) {
        x_ = xbc[static_cast<size_t>(t) * ldx + h * P + pc];
        d_ = raw_dt[static_cast<size_t>(t) * ldd + h];
        const float* Bt = b_row + static_cast<size_t>(t) * ldx;
        const float* Ct = c_row + static_cast<size_t>(t) * ldx;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            B_[j] = Bt[min(j, nn - 1)];
            C_[j] = Ct[min(j, nn - 1)];
        }
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            B_[j] = j < nn ? B_[j] : 0.f;
            C_[j] = j < nn ? C_[j] : 0.f;
        }
    };
    load(min(t0, t1 - 1), xv, dtr, Bv, Cv);
    float cum = 0.f;
    for (int t = t0; t < t1; ++t) {
        float xn, dn, Bn[NS], Cn[NS];
        load(min(t + 1, t1 - 1), xn, dn, Bn, Cn);
        const float dt = softplus_precise(dtr + bias);
        const float a = expf(neg_rate * dt), dx = dt * xv;
        cum += neg_rate * dt;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            S[j] = a * S[j] + dx * Bv[j];
            acc += S[j] * Cv[j];
        }
        if (p_ok) yp[static_cast<size_t>(t) * ldy] = acc + skip * xv;
        if (co.n_chunks > 1 && blockIdx.x == 0 && lane == 0) cumlog[static_cast<size_t>(t) * H + h] = cum;
        xv = xn; dtr = dn;
#pragma unroll
        for (int j = 0; j < NS; ++j) { Bv[j] = Bn[j]; Cv[j] = Cn[j]; }
    }
    if (!p_ok) return;
    if (co.n_chunks > 1) sp = chunk_state + ((static_cast<size_t>(co.first_chunk + co.k) * H + h) * N + n0) * P + p;
    if (write || co.n_chunks > 1) {
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (j < nn) sp[static_cast<size_t>(j) * P] = S[j];
    }
}

// The same scan with the chunk's operands staged in LDS first: x [chunk][64], B and C of the slice [chunk][NS]
// and the raw step sizes, all requested at once with 16-byte loads, so that the token loop waits for no memory
// (one token ahead is not enough to cover a load that another XCD's kernel wrote a moment ago). Needs 16-byte
// aligned rows and column offsets (the launcher checks) and chunk <= CH.
template <int NS, int CH>
__global__ void __launch_bounds__(64)
ssm_scan_staged_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ raw_dt, int ldd,
                       const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
                       const int* __restrict__ cu_q, const int* __restrict__ state_slots, int n_seqs, float* __restrict__ state,
                       size_t slot_floats, size_t scan_offset, float* __restrict__ y, int ldy, size_t part_stride, int H, int P,
                       int N, int G, int n_slices, int write, int chunk, float* __restrict__ chunk_state,
                       float* __restrict__ cumlog) {
    __shared__ __attribute__((aligned(16))) float xs[CH][64];
    __shared__ __attribute__((aligned(16))) float Bs[CH][NS];
    __shared__ __attribute__((aligned(16))) float Cs[CH][NS];
    __shared__ float dts[64], as[64];                 // step size and decay of the chunk's tokens
    const int lane = threadIdx.x;
    const int h = blockIdx.y, slice = blockIdx.x % n_slices, p0 = (blockIdx.x / n_slices) * 64, p = p0 + lane;
    const ChunkOf co = chunk_of(blockIdx.z, cu_q, n_seqs, chunk, chunk_state != nullptr);
    if (co.b < 0) return;
    const int slot = state_slots[co.b];
    if (slot < 0) return;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int n0 = slice * NS, nn = min(NS, N - n0);
    const int t0 = cu_q[co.b] + co.k * chunk, t1 = min(t0 + chunk, cu_q[co.b + 1]), nt = t1 - t0;
    float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * N + n0) * P + pc;
    float S[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = sp[static_cast<size_t>(min(j, nn - 1)) * P];
    // Staging: quads of 4 floats, a fixed number per lane (CH * 16 quads of x, CH * NS / 4 of B and of C over 64
    // lanes), all requested before the first is written to LDS; tokens beyond the chunk's end repeat its last one,
    // a quad beyond the row's end (P or N no multiple of the tile) the row's last one.
    const int pq = min(64, P - p0) / 4, nq = nn / 4;           // whole quads of x and of B, C in this tile
    {
        float4 xq[CH / 4];
#pragma unroll
        for (int u = 0; u < CH / 4; ++u) {
            const int e = lane + 64 * u, tt = min(e / 16, nt - 1), q = min(e % 16, pq - 1);
            xq[u] = *reinterpret_cast<const float4*>(xbc + static_cast<size_t>(t0 + tt) * ldx + h * P + p0 + 4 * q);
        }
        constexpr int BQ = CH * (NS / 4) / 64;
        float4 bq[BQ], cq[BQ];
#pragma unroll
        for (int u = 0; u < BQ; ++u) {
            const int e = lane + 64 * u, tt = min(e / (NS / 4), nt - 1), q = min(e % (NS / 4), nq - 1);
            const float* row = xbc + static_cast<size_t>(t0 + tt) * ldx + inner + g * N + n0 + 4 * q;
            bq[u] = *reinterpret_cast<const float4*>(row);
            cq[u] = *reinterpret_cast<const float4*>(row + G * N);
        }
#pragma unroll
        for (int u = 0; u < CH / 4; ++u) {
            const int e = lane + 64 * u;
            *reinterpret_cast<float4*>(&xs[e / 16][4 * (e % 16)]) = xq[u];
        }
#pragma unroll
        for (int u = 0; u < BQ; ++u) {
            const int e = lane + 64 * u, qi = e % (NS / 4);
            const bool real = qi < nq;                          // rows of the slice beyond N count as zeros
            *reinterpret_cast<float4*>(&Bs[e / (NS / 4)][4 * qi]) = real ? bq[u] : make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4*>(&Cs[e / (NS / 4)][4 * qi]) = real ? cq[u] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    // Step sizes and decays are the same for every lane: lane t works them out for token t of the chunk, once
    // (softplus, two exponentials), and a running sum over the lanes gives the logarithm of the decay accumulated
    // since the chunk began.
    const float bias = dt_bias[h], neg_rate = -expf(A_log[h]), skip = slice == 0 ? Dskip[h] : 0.f;
    {
        static_assert(CH <= 64, "one lane per token of a chunk");
        const float dt = softplus_precise(raw_dt[static_cast<size_t>(t0 + min(lane, nt - 1)) * ldd + h] + bias);
        const float lg = lane < nt ? neg_rate * dt : 0.f;
        float run = lg;
#pragma unroll
        for (int off = 1; off < 64; off *= 2) {
            const float up = __shfl_up(run, off, 64);
            if (lane >= off) run += up;
        }
        dts[lane] = dt;
        as[lane] = expf(lg);
        if (co.n_chunks > 1 && blockIdx.x == 0 && lane < nt) cumlog[static_cast<size_t>(t0 + lane) * H + h] = run;
    }
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = (co.k == 0 && j < nn) ? S[j] : 0.f;
    float* yp = y + slice * part_stride + h * P + pc;
    wave_lds_sync();
    for (int tt = 0; tt < nt; ++tt) {
        const float xv = xs[tt][lane];
        const float a = as[tt], dx = dts[tt] * xv;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NS; j += 4) {
            const float4 b4 = *reinterpret_cast<const float4*>(&Bs[tt][j]), c4 = *reinterpret_cast<const float4*>(&Cs[tt][j]);
            S[j] = a * S[j] + dx * b4.x;         acc[0] += S[j] * c4.x;
            S[j + 1] = a * S[j + 1] + dx * b4.y; acc[1] += S[j + 1] * c4.y;
            S[j + 2] = a * S[j + 2] + dx * b4.z; acc[2] += S[j + 2] * c4.z;
            S[j + 3] = a * S[j + 3] + dx * b4.w; acc[3] += S[j + 3] * c4.w;
        }
        if (p_ok) yp[static_cast<size_t>(t0 + tt) * ldy] = (acc[0] + acc[1]) + (acc[2] + acc[3]) + skip * xv;
    }
    if (!p_ok) return;
    if (co.n_chunks > 1) sp = chunk_state + ((static_cast<size_t>(co.first_chunk + co.k) * H + h) * N + n0) * P + p;
    if (write || co.n_chunks > 1) {
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (j < nn) sp[static_cast<size_t>(j) * P] = S[j];
    }
}

// What the chunks before chunk k of a portion contribute to it (see ssm_scan_kernel): with A_j the whole
// decay of chunk j and L_j its last local state, the state at the start of chunk k is
//   S = L_0 for k = 1;  S <- A_j S + L_j for j = 1 .. k - 1,
// every token t of chunk k gets  y[t] += exp(cumlog[t]) sum_n C[t, n] S[n, p] (slice by slice, as the scan), and
// the portion's last chunk writes A_k S + L_k back to the slot. Same grid and lane layout as the scan.
template <int NS>
__global__ void __launch_bounds__(64)
ssm_chunk_join_kernel(const float* __restrict__ xbc, int ldx, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                      int n_seqs, float* __restrict__ state, size_t slot_floats, size_t scan_offset, float* __restrict__ y,
                      int ldy, size_t part_stride, int H, int P, int N, int G, int n_slices, int write, int chunk,
                      const float* __restrict__ chunk_state, const float* __restrict__ cumlog) {
    const int lane = threadIdx.x;
    const int h = blockIdx.y, slice = blockIdx.x % n_slices, p = (blockIdx.x / n_slices) * 64 + lane;
    const ChunkOf co = chunk_of(blockIdx.z, cu_q, n_seqs, chunk, true);
    if (co.b < 0 || co.k == 0) return;                         // surplus, or a first chunk: nothing comes before it
    const int slot = state_slots[co.b];
    if (slot < 0) return;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int n0 = slice * NS, nn = min(NS, N - n0);
    const int q0 = cu_q[co.b], q1 = cu_q[co.b + 1];
    auto local_state = [&](int j) { return chunk_state + ((static_cast<size_t>(co.first_chunk + j) * H + h) * N + n0) * P + pc; };
    auto chunk_decay = [&](int j) { return expf(cumlog[static_cast<size_t>(min(q0 + (j + 1) * chunk, q1) - 1) * H + h]); };
    // (loads without conditions, from clamped indices, as in the scan; rows of the slice beyond N stay zero)
    float S[NS];
    {
        const float* l0 = local_state(0);
#pragma unroll
        for (int j = 0; j < NS; ++j) S[j] = l0[static_cast<size_t>(min(j, nn - 1)) * P];
#pragma unroll
        for (int j = 0; j < NS; ++j) S[j] = j < nn ? S[j] : 0.f;
    }
    for (int c = 1; c < co.k; ++c) {
        const float a = chunk_decay(c);
        const float* lc = local_state(c);
        float L[NS];
#pragma unroll
        for (int j = 0; j < NS; ++j) L[j] = lc[static_cast<size_t>(min(j, nn - 1)) * P];
#pragma unroll
        for (int j = 0; j < NS; ++j) S[j] = j < nn ? a * S[j] + L[j] : 0.f;
    }
    const int t0 = q0 + co.k * chunk, t1 = min(t0 + chunk, q1);
    const float* c_row = xbc + inner + G * N + g * N + n0;
    float* yp = y + slice * part_stride + h * P + pc;
    // the chunk's C rows of the slice and its tokens' decays go to LDS first, all requested at once (as the scan
    // stages its operands); y is then read, added to and written sixteen tokens at a time
    __shared__ float Cs[64][NS + 1];
    __shared__ float seen_s[64];
    const int nt = t1 - t0;
    {
        float cv[NS];
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const int e = lane + 64 * u, tt = min(e / NS, nt - 1), j = min(e % NS, nn - 1);
            cv[u] = c_row[static_cast<size_t>(t0 + tt) * ldx + j];
        }
        const float sv = cumlog[static_cast<size_t>(t0 + min(lane, nt - 1)) * H + h];
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const int e = lane + 64 * u;
            Cs[e / NS][e % NS] = cv[u];
        }
        seen_s[lane] = expf(sv);
    }
    wave_lds_sync();
    for (int t = 0; t < nt; t += 16) {
        float before[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) before[u] = yp[static_cast<size_t>(t0 + min(t + u, nt - 1)) * ldy];     // (pc is a valid column for every lane)
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int tt = min(t + u, nt - 1);
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < NS; ++j) acc += S[j] * Cs[tt][j];         // (S is zero beyond N)
            if (p_ok && t + u < nt) yp[static_cast<size_t>(t0 + t + u) * ldy] = before[u] + seen_s[tt] * acc;
        }
    }
    if (write && co.k == co.n_chunks - 1) {
        const float a = chunk_decay(co.k);
        const float* lk = local_state(co.k);
        float L[NS];
#pragma unroll
        for (int j = 0; j < NS; ++j) L[j] = lk[static_cast<size_t>(min(j, nn - 1)) * P];
        float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * N + n0) * P + pc;
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (j < nn && p_ok) sp[static_cast<size_t>(j) * P] = a * S[j] + L[j];
    }
}

}  // namespace

// The launch of rmsnorm_conv_single_kernel by taps, width and output type.
template <int MODE>
static int stream_conv_single_launch(float* x, int ldx, const float* y, int ldy, const float* wn, float eps, int C, const float* wc,
                                     int taps, const int* state_slots, float* state, size_t slot_floats, void* out, int ldo,
                                     int out_dtype, int T, int write, hipStream_t stream) {
#define RCS(TYPE, TAPS, NB)                                                                                            \
    rmsnorm_conv_single_kernel<TYPE, TAPS, NB, MODE><<<T, 64 * NB, 0, stream>>>(x, ldx, y, ldy, wn, eps, C, wc, state_slots, state, \
                                                                               slot_floats, static_cast<TYPE*>(out), ldo, write)
#define RCS_NB(TYPE, TAPS)                                                                                             \
    do {                                                                                                               \
        if (C <= 512) RCS(TYPE, TAPS, 1); else if (C <= 1024) RCS(TYPE, TAPS, 2); else if (C <= 1536) RCS(TYPE, TAPS, 3);   \
        else RCS(TYPE, TAPS, 4);                                                                                       \
    } while (0)
#define RCS_TAPS(TYPE)                                                                                                 \
    switch (taps) {                                                                                                    \
        case 1: RCS_NB(TYPE, 1); break; case 2: RCS_NB(TYPE, 2); break; case 3: RCS_NB(TYPE, 3); break;                \
        case 4: RCS_NB(TYPE, 4); break; case 5: RCS_NB(TYPE, 5); break; case 6: RCS_NB(TYPE, 6); break;                \
        case 7: RCS_NB(TYPE, 7); break; default: RCS_NB(TYPE, 8); break;                                               \
    }
    if (out_dtype == MLLM_F32) { RCS_TAPS(float) } else { RCS_TAPS(bf16_t) }
#undef RCS_TAPS
#undef RCS_NB
#undef RCS
    MLLM_LAUNCH_CHECK();
    return 0;
}

extern "C" {

// Convolution + silu of columns [col0, col0 + C) of proj's rows into out [T, C]; then, with `write`, the
// slots' carried rows are brought up to date (a second kernel: it overwrites what the first one reads).
// -1: taps outside 1..16.
int mllm_conv_silu(const float* proj, int ld, int col0, int C, const float* w, const float* bias, int taps,
                   const int* token_seq, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                   float* out, int ldo, int T, int B, int write, hipStream_t stream) {
    if (T <= 0 || C <= 0) return 0;
    if (taps < 1 || taps > 16) return -1;
    const long long total = static_cast<long long>(T) * C;
    // (one token a sequence: the convolution's kernel brings the carried rows up to date itself)
    const bool single = T == B && write && taps > 1;
    conv_silu_kernel<<<static_cast<int>((total + 255) / 256), 256, 0, stream>>>(proj, ld, col0, C, w, bias, taps, token_seq, cu_q,
                                                                                state_slots, state, slot_floats, out, ldo, total, single ? 1 : 0);
    MLLM_LAUNCH_CHECK();
    if (write && taps > 1 && !single) {
        const long long pairs = static_cast<long long>(B) * C;
        conv_carry_kernel<<<static_cast<int>((pairs + 255) / 256), 256, 0, stream>>>(proj, ld, col0, C, taps, cu_q, state_slots, state,
                                                                                    slot_floats, B);
        MLLM_LAUNCH_CHECK();
    }
    return 0;
}

// out = in + conv(in) (residual == 0: conv(in) alone) over the C columns of in's rows (fp32), out in out_dtype; the
// slots' carried rows are brought up to date as by mllm_conv_silu. -1: taps outside 1..16.
int mllm_conv_residual(const float* in, int ld, int C, const float* w, int taps, const int* token_seq, const int* cu_q,
                       const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                       int B, int write, hipStream_t stream, int residual) {
    if (T <= 0 || C <= 0) return 0;
    if (taps < 1 || taps > 16) return -1;
    const long long total = static_cast<long long>(T) * C;
    const bool single = T == B && write && taps > 1;
    const bool vec = taps <= 8 && C % 4 == 0 && ld % 4 == 0 && ldo % 4 == 0 && slot_floats % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(state) |
                       reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (vec) {
        const long long total4 = total / 4;
        const int blocks4 = static_cast<int>((total4 + 255) / 256);
#define CRV(TYPE, TAPS)                                                                                                \
    conv_residual_vec_kernel<TYPE, TAPS><<<blocks4, 256, 0, stream>>>(in, ld, C, w, token_seq, cu_q, state_slots, state, slot_floats, \
                                                                     static_cast<TYPE*>(out), ldo, total4, single ? 1 : 0, residual)
#define CRV_TAPS(TYPE)                                                                                                 \
    switch (taps) {                                                                                                    \
        case 1: CRV(TYPE, 1); break; case 2: CRV(TYPE, 2); break; case 3: CRV(TYPE, 3); break; case 4: CRV(TYPE, 4); break; \
        case 5: CRV(TYPE, 5); break; case 6: CRV(TYPE, 6); break; case 7: CRV(TYPE, 7); break; default: CRV(TYPE, 8); break; \
    }
        if (out_dtype == MLLM_F32) { CRV_TAPS(float) } else { CRV_TAPS(bf16_t) }
#undef CRV_TAPS
#undef CRV
    } else {
        const int blocks = static_cast<int>((total + 255) / 256);
        if (out_dtype == MLLM_F32)
            conv_residual_kernel<float><<<blocks, 256, 0, stream>>>(in, ld, C, w, taps, token_seq, cu_q, state_slots, state, slot_floats,
                                                                    static_cast<float*>(out), ldo, total, single ? 1 : 0, residual);
        else
            conv_residual_kernel<bf16_t><<<blocks, 256, 0, stream>>>(in, ld, C, w, taps, token_seq, cu_q, state_slots, state,
                                                                     slot_floats, static_cast<bf16_t*>(out), ldo, total, single ? 1 : 0, residual);
    }
    MLLM_LAUNCH_CHECK();
    if (write && taps > 1 && !single) {
        const long long pairs = static_cast<long long>(B) * C;
        conv_carry_kernel<<<static_cast<int>((pairs + 255) / 256), 256, 0, stream>>>(in, ld, 0, C, taps, cu_q, state_slots, state,
                                                                                    slot_floats, B);
        MLLM_LAUNCH_CHECK();
    }
    return 0;
}

// out = h + conv(h), h = rmsnorm(x) * wn, for a step of T sequences of one token each (token t is sequence t).
// -1: taps outside 1..16; -2: more than 8 taps or rows of more than 2,048 columns (nothing is launched).
int mllm_rmsnorm_conv_single(const float* x, int ldx, const float* wn, float eps, int C, const float* wc, int taps,
                             const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                             int write, hipStream_t stream) {
    if (T <= 0 || C <= 0) return 0;
    if (taps < 1 || taps > 16) return -1;
    if (taps > 8 || C > 2048) return -2;           // sizes this kernel is not made for: norm and convolution apart
    // (this mode only reads x)
    return stream_conv_single_launch<0>(const_cast<float*>(x), ldx, nullptr, 0, wn, eps, C, wc, taps, state_slots, state, slot_floats, out,
                                        ldo, out_dtype, T, write, stream);
}

// For a step of T sequences of one token each, the stream's rows x [T, C] (fp32) and a block's input convolution:
// with y (a sub-layer's result, fp32 [T, C]) and wn: x += y / sqrt(mean(y^2) + eps) * wn first (x is written), then
// out = x + conv(x); with y null: out = x + conv(x) alone. Return codes as mllm_rmsnorm_conv_single's.
int mllm_stream_conv_single(float* x, int ldx, const float* y, int ldy, const float* wn, float eps, int C, const float* wc, int taps,
                            const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                            int write, hipStream_t stream) {
    if (T <= 0 || C <= 0) return 0;
    if (taps < 1 || taps > 16 || (y != nullptr && wn == nullptr)) return -1;
    if (taps > 8 || C > 2048) return -2;
    if (y != nullptr)
        return stream_conv_single_launch<1>(x, ldx, y, ldy, wn, eps, C, wc, taps, state_slots, state, slot_floats, out, ldo, out_dtype, T,
                                            write, stream);
    return stream_conv_single_launch<2>(x, ldx, nullptr, 0, nullptr, eps, C, wc, taps, state_slots, state, slot_floats, out, ldo,
                                        out_dtype, T, write, stream);
}

// Tokens of a chunk, rows of n a wavefront keeps, and what the chunks' workspace must hold for a step of T tokens.
#define SSM_CHUNK 64
#define SSM_SLICE 32
static size_t chunk_states(int T) { return 2 * static_cast<size_t>(T) / SSM_CHUNK + 1; }
size_t mllm_ssm_scan_workspace_floats(int T, int B, int H, int P, int N) {
    (void)B;
    return chunk_states(T) * H * P * N + static_cast<size_t>(T) * H;
}
// The scan leaves y as this many shares (see ssm_scan_kernel), part_stride floats apart.
int mllm_ssm_scan_parts(int N) { return (N + SSM_SLICE - 1) / SSM_SLICE; }

// The scan over every sequence's portion (see the kernels). `workspace` (mllm_ssm_scan_workspace_floats floats)
// is needed when a portion is longer than one chunk (max_q_len > 64). -1: H is no multiple of G, or the
// workspace is missing.
int mllm_ssm_scan(const float* xbc, int ldx, const float* raw_dt, int ldd, const float* dt_bias, const float* A_log,
                  const float* Dskip, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                  size_t scan_offset, float* y, int ldy, size_t part_stride, int T, int B, int max_q_len, int H, int P, int N,
                  int G, int write, float* workspace, hipStream_t stream) {
    if (B <= 0 || T <= 0) return 0;
    if (H < 1 || G < 1 || H % G != 0 || N < 1 || P < 1) return -1;
    const bool chunked = max_q_len > SSM_CHUNK;
    if (chunked && workspace == nullptr) return -1;
    const int n_chunks = chunked ? T / SSM_CHUNK + B : B;
    float* chunk_state = workspace;
    float* cumlog = workspace ? workspace + chunk_states(T) * H * P * N : nullptr;
    const int n_slices = mllm_ssm_scan_parts(N);
    const dim3 grid(((P + 63) / 64) * n_slices, H, n_chunks);
    const bool aligned = ldx % 4 == 0 && P % 4 == 0 && N % 4 == 0 && (reinterpret_cast<uintptr_t>(xbc) & 15) == 0;
    if (aligned)
        ssm_scan_staged_kernel<SSM_SLICE, SSM_CHUNK><<<grid, 64, 0, stream>>>(xbc, ldx, raw_dt, ldd, dt_bias, A_log, Dskip, cu_q, state_slots,
                                                                             B, state, slot_floats, scan_offset, y, ldy, part_stride, H, P, N,
                                                                             G, n_slices, write, SSM_CHUNK, chunked ? chunk_state : nullptr,
                                                                             cumlog);
    else
        ssm_scan_kernel<SSM_SLICE><<<grid, 64, 0, stream>>>(xbc, ldx, raw_dt, ldd, dt_bias, A_log, Dskip, cu_q, state_slots, B, state,
                                                           slot_floats, scan_offset, y, ldy, part_stride, H, P, N, G, n_slices, write,
                                                           SSM_CHUNK, chunked ? chunk_state : nullptr, cumlog);
    if (chunked)
        ssm_chunk_join_kernel<SSM_SLICE><<<grid, 64, 0, stream>>>(xbc, ldx, cu_q, state_slots, B, state, slot_floats, scan_offset, y,
                                                                 ldy, part_stride, H, P, N, G, n_slices, write, SSM_CHUNK,
                                                                 chunk_state, cumlog);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
