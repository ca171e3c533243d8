// The engine's device operations: checked dispatch over the HIP kernels.
//
// Every op checks on the host that shapes, strides and dtypes are what the kernel it picks and
// that kernel's grid assume, chooses among the kernels of an operation by size, and launches on
// the stream it is given. A refusal is an OpError
// with a message that names the sizes. There is no CPU path.
//
// The parts (parts.h) and, through the C ABI, the kernel tests (kernels/ops.py) call the same
// functions, so the choice of kernels is made in one place.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "score_shape.h"

namespace minillm {

enum DType : int { F32 = 0, BF16 = 1 };
inline size_t dtype_size(int dt) { return dt == F32 ? 4 : 2; }
const char* dtype_name(int dt);

enum Epilogue : int { STORE = 0, GELU_TANH = 1, GELU_ERF = 2, ADD_RESIDUAL = 3, STORE_F32 = 4 };
// Activations that only the gated feed-forward's kernel knows (glu_act), beside GELU_TANH.
enum GluActivation : int { GLU_SILU = 5 };

class OpError : public std::runtime_error {
public:
    explicit OpError(const std::string& what) : std::runtime_error(what) {}
};
[[noreturn]] void fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// A 2-D view of device memory; the last dimension is contiguous, `stride` elements lie between rows.
struct Tensor2 {
    void* data = nullptr;
    int dtype = F32;
    int64_t rows = 0, cols = 0, stride = 0;

    Tensor2() = default;
    Tensor2(void* d, int dt, int64_t r, int64_t c) : data(d), dtype(dt), rows(r), cols(c), stride(c) {}
    Tensor2(void* d, int dt, int64_t r, int64_t c, int64_t s) : data(d), dtype(dt), rows(r), cols(c), stride(s) {}
    size_t esz() const { return dtype_size(dtype); }
    bool contiguous() const { return stride == cols; }
    Tensor2 row_range(int64_t first, int64_t n) const {
        return Tensor2(static_cast<char*>(data) + first * stride * static_cast<int64_t>(esz()), dtype, n, cols, stride);
    }
};

// Second destination of a fused QKV product: the columns after the first q_cols are keys, then
// values (kv_dim = k_pages.cols each); row m's also go to row slots[m] (>= 0) of the pages.
struct KvScatter {
    const int* slots = nullptr;
    Tensor2 k_pages, v_pages;
    int q_cols = 0;
};

// The output of decode attention that has not been merged yet: every (token, head) pair's keys were
// split over `nsplit` workgroups whose states lie in the attention scratch (layout:
// kernels/attention_decode.hip). `linear_from_splits` merges while it loads. Valid until the next
// attention launch on the same stream.
struct AttentionSplits {
    float* ws = nullptr;
    int n_tokens = 0, n_heads = 0, head_dim = 0, nsplit = 0, dtype = BF16;
    bool valid() const { return ws != nullptr; }
    float* ml() const { return ws + static_cast<size_t>(n_tokens) * n_heads * nsplit * head_dim; }
};

struct AttentionArgs {
    Tensor2 q;                     // [T, >= q_col + n_heads * head_dim]
    int q_col = 0, n_heads = 0, n_kv_heads = 0, head_dim = 0;
    Tensor2 k_pages, v_pages;      // [n_pages * page_size, n_kv_heads * head_dim]
    int page_size = 0;
    const int* block_tables = nullptr;     // [n_seqs, max_blocks]
    int n_seqs = 0, max_blocks = 0;
    const int* token_seq = nullptr;        // [T] row of block_tables
    const int* positions = nullptr;        // [T]
    float scale = 1.f;
    int window = 0;
    Tensor2 out;                   // [T, n_heads * head_dim]
    const int* cu_q = nullptr;     // [n_seqs + 1] (needed by the query-tile kernel)
    const int* ctx_len = nullptr;  // [n_seqs]
    int max_q_len = 0, max_ctx_len = 0;
    int append = 0;                // != 0: the step's keys/values are still in q's rows: write them to the pages first
    int k_col = 0, v_col = 0;
    const int* slots = nullptr;    // [T] rows of the pages (append)
    int n_single = 0;              // the first n_single sequences bring one token each
    int may_split = 0;             // != 0: the caller takes an AttentionSplits in place of `out`
    // scores shaped before the softmax and a chunked mask (score_shape.h), or null; and a gate: the result is
    // multiplied by sigmoid(gate[t, gate_col + column]) (fp32 rows, row stride gate_stride). Neither goes with may_split.
    const MllmScoreShape* shape = nullptr;
    const float* gate = nullptr;
    int gate_stride = 0;
};

// -- scratch: device memory that kernels need beyond inputs and outputs, one set per stream -----------
// Work on one stream runs in order, so the kernels launched on it can share these buffers; two runners
// (two streams) never share one, so their steps may overlap on the device. A part says what its kernels
// need through the reserve_* calls when its runner is built, so that no step allocates; an op that is
// called with more than was reserved (tests call ops directly) grows the buffer, which synchronises the
// device. release_scratch frees a stream's buffers (the owner of the stream calls it before it destroys it).
void reserve_attention_scratch(int rows, int n_heads, int head_dim, hipStream_t stream);
void reserve_sampling_scratch(int rows, int vocab, hipStream_t stream);
void reserve_linear_scratch(hipStream_t stream);
void release_scratch(hipStream_t stream);
void* scratch_address(const char* name, hipStream_t stream);      // nullptr if not allocated yet (tests)
size_t scratch_bytes();                                            // all streams of the current device (tests)

// -- tuning hooks (tests and tuning scripts) ---------------------------------------------------------
struct Tuning {
    int decode_nsplit = 0, decode_waves = 0;          // > 0: forced launch shape of merged decode attention
    int unmerged_nsplit = 0, unmerged_waves = 0;      // > 0: forced shape of splits merged by the next product
    int merge_max_rows = 16;                          // tokens whose splits a product merges while loading
    int long_context_splits = 1;                      // 1: few pairs with long contexts are split over up to 256 workgroups
    int ln_fuse_max_rows = 32;                        // rows up to which the norm is fused into the few-row product
    int latent_tiles = 1;                             // 1: latent attention's prompt portions may run on the matrix cores
    int scored_shared_kernels = 1;                    // 1: attention with shaped scores may run on the kernels the plain attention runs on
    int halves_max_width = 1024;                      // stream widths up to which a block whose sub-layers read one stream runs the
                                                      // feed-forward's first products, with the norm inside, in front of the mixer
                                                      // (wider: every workgroup of a wide product redoing the norm costs more than the
                                                      // norm's own kernel; at width 1,600 the halves lost 5 % of a decode step)
    // what the ops chose since the last reset (tests read it back instead of trusting the thresholds)
    struct Seen {
        int max_decode_splits = 0;                    // most workgroups a (token, head) pair's keys were split over
        long long merge_kernel_launches = 0, prefill_tile_launches = 0, tiled_f32_launches = 0, generic_attention_launches = 0;
        long long latent_tile_launches = 0, latent_token_launches = 0;      // latent attention: matrix-core kernel, one workgroup per token
    } seen;
};
Tuning& tuning();

// Token ids that an earlier step sampled on the device and the host has not read yet: where src[t] >= 0,
// token t's id is prev[src[t]] (n_prev entries) and not ids[t].
struct FedTokens {
    const int* src = nullptr;
    const int* prev = nullptr;
    int n_prev = 0;
};

// -- the ops -----------------------------------------------------------------------------------------
// out[t, :] = scale * wte[ids[t], :] (+ wpe[positions[t], :])
void embed(const int* ids, const int* positions, const Tensor2& wte, const Tensor2* wpe, const Tensor2& out,
           hipStream_t stream, const FedTokens* fed = nullptr, float scale = 1.f);
void select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream);
void reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int n_seqs,
                 hipStream_t stream);
// out[i,:] = LayerNorm(x[rows ? rows[i] : i, :]); out.rows rows.
void layernorm(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& out,
               const int* rows, hipStream_t stream);
void kv_append(const Tensor2& src, int k_col, int v_col, const Tensor2& k_pages, const Tensor2& v_pages,
               const int* slots, hipStream_t stream);
// out = epilogue(a w^T + bias); a [M,K], w [N,K] of one dtype, bias fp32 [N] or null.
void linear(const Tensor2& a, const Tensor2& w, const float* bias, const Tensor2& out, int epilogue,
            const KvScatter* kv, hipStream_t stream);
// The same with a = the merged attention splits. `tmp` ([n_tokens, n_heads*head_dim] in w's dtype) is
// used only if the merging kernel does not take these sizes (then: merge kernel, ordinary product).
void linear_from_splits(const AttentionSplits& a, const Tensor2& w, const float* bias, const Tensor2& out,
                        int epilogue, void* tmp, hipStream_t stream);
void merge_splits(const AttentionSplits& a, const Tensor2& out, hipStream_t stream);
// out = epilogue(LayerNorm(x[rows]) w^T + bias), the norm fused into the product where the kernels allow;
// `tmp` ([out.rows, K] in w's dtype) holds the normalised rows otherwise. `kv` as for linear.
void ln_linear(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& w,
               const float* bias, const Tensor2& out, int epilogue, const int* rows, void* tmp,
               const KvScatter* kv, hipStream_t stream);
// Causal attention of the step's queries over the pages. Returns true and fills *splits when the result is
// left unmerged (only with may_split); otherwise `out` holds it.
bool paged_attention(const AttentionArgs& a, AttentionSplits* splits, hipStream_t stream);

// -- RMS norms, gated activation ---------------------------------------------------------------------
// out[i, :] = x[rows ? rows[i] : i, :] / sqrt(mean(.^2) + eps) * weight, the columns in `groups` equal parts
// that are normed one by one; with `gate` (fp32, x's shape) the input is x * silu(gate) (the gate comes
// before the norm). x fp32 (any row stride), out in its own dtype. With parts > 1 the input is the sum of `parts`
// arrays of x's shape that lie part_stride floats apart (x the first), added in the order of their index.
void rmsnorm(const Tensor2& x, const float* weight, float eps, int groups, const Tensor2* gate, const Tensor2& out,
             const int* rows, hipStream_t stream, int parts = 1, size_t part_stride = 0);
// out = epilogue(rmsnorm(x[rows]) w^T + bias), the norm inside the product where the kernels allow (bfloat16, few
// rows); `tmp` ([out.rows, K] in w's dtype) holds the normalised rows otherwise.
void rms_linear(const Tensor2& x, const float* weight, float eps, const Tensor2& w, const float* bias, const Tensor2& out,
                int epilogue, const int* rows, void* tmp, hipStream_t stream);
// x += mult * scale * (y / sqrt(mean(y^2) + eps) * weight), row by row (scale: per column, or null);
// `clear`: y is zero afterwards.
void rmsnorm_add(const Tensor2& y, const float* weight, const float* scale, float mult, float eps, const Tensor2& x,
                 bool clear, hipStream_t stream);
// out = g sigmoid(alpha g) (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit)
void glu_clamped(const Tensor2& gate, const Tensor2& up, float limit, float alpha, const Tensor2& out, hipStream_t stream);
void fill_zero(const Tensor2& x, hipStream_t stream);          // contiguous fp32, by a kernel

// -- state-space mixer -------------------------------------------------------------------------------
// A step's sequences with per-request state slots ([n_slots, slot_floats] fp32).
struct StateArgs {
    const int* token_seq = nullptr;    // [T]
    const int* cu_q = nullptr;         // [B + 1]
    const int* state_slots = nullptr;  // [B], < 0: padding
    int n_seqs = 0, max_q_len = 0;     // max_q_len: the longest portion of the step
    float* state = nullptr;
    size_t slot_floats = 0;
    int n_slots = 0;
    bool write = true;
};
// out[t, :] = silu(conv(columns [col0, col0 + C) of proj)), causal per sequence over `taps` inputs, the inputs
// before a portion taken from the slot's first (taps - 1) * C floats, which are brought up to date afterwards.
void conv_silu(const Tensor2& proj, int col0, const Tensor2& weight, const float* bias, const StateArgs& st,
               const Tensor2& out, hipStream_t stream);
// The Mamba-2 scan (kernels/ssm.hip) over xbc [T, H*P + 2*G*N] and the raw step sizes (columns dt_col.. of
// proj), state at `scan_offset` floats into the slot. y comes as ssm_scan_parts(N) shares, each [T, H*P] fp32
// and y.rows * y.stride floats after the one before (y is the first); their sum in the order of their index is
// the result (rmsnorm adds them while it reads). Portions longer than a chunk are scanned chunk by chunk side by
// side and joined, for which `workspace` (ssm_scan_workspace_floats floats) is needed.
void ssm_scan(const Tensor2& xbc, const Tensor2& proj, int dt_col, const float* dt_bias, const float* A_log,
              const float* skip, const StateArgs& st, size_t scan_offset, int H, int P, int N, int G, const Tensor2& y,
              float* workspace, size_t workspace_floats, hipStream_t stream);
size_t ssm_scan_workspace_floats(int tokens, int n_seqs, int H, int P, int N);
int ssm_scan_parts(int N);

// -- latent attention --------------------------------------------------------------------------------
struct LatentShape {
    int n_heads = 0, plain_dim = 0, rot_dim = 0, value_dim = 0, kv_rank = 0, q_rank = 0, rot_dims = 0;
    double rot_base = 10000.0;
    float eps = 1e-6f;
};
// The pages of latent attention: `rows` [n_pages * page_size, kv_rank + rot_dim] holds a row [c | k_rot] per
// token; `latent_t` (optional, [n_pages * page_size, kv_rank] in size) holds c once more, transposed page by
// page ([page][kv_rank][page_size]): the operand shape of the matrix-core kernel.
struct LatentPages {
    Tensor2 rows, latent_t;
    int page_size = 0;
};
// cq = rmsnorm(dq) * wq; with dkv: page row slots[t] = [rmsnorm(dkv[:, :kv_rank]) * wkv | turned rest]
void latent_prepare(const Tensor2& dq, const float* wq, const Tensor2& cq, const Tensor2* dkv, const float* wkv,
                    const LatentPages* pages, const int* slots, const int* positions, const LatentShape& sh, hipStream_t stream);
// qa[t, h] = [W_uk_h^T q_plain[t, h] | turned q_rot[t, h]]; w_uk is handed over transposed, [kv_rank, heads * plain_dim]
void latent_absorb(const Tensor2& q, const Tensor2& w_uk, const Tensor2& qa, const int* positions, const LatentShape& sh,
                   hipStream_t stream);
// The step's sequences, as attention sees them.
struct LatentStep {
    const int* block_tables = nullptr;     // [n_seqs, max_blocks]
    int max_blocks = 0, n_seqs = 0, max_q_len = 0, max_ctx_len = 0;
    const int* token_seq = nullptr;        // [T]
    const int* positions = nullptr;        // [T]
    const int* cu_q = nullptr;             // [n_seqs + 1]
    const int* ctx_len = nullptr;          // [n_seqs]
};
// o_lat[t, h] = sum_j softmax_j(scale * qa[t, h] . row_j) row_j[:kv_rank] over the visible rows of the pages.
// Runs on the matrix cores where the sizes allow (bfloat16, the transposed latent at hand), otherwise one
// workgroup per token. `workspace` (optional, fp32, latent_attention_workspace_floats(...) floats): steps of few
// rows (decoding) then spread every row's keys over several workgroups, whose states meet there.
void latent_attention(const Tensor2& qa, const LatentPages& pages, const LatentStep& step, float scale, int window,
                      const LatentShape& sh, const Tensor2& o_lat, float* workspace, size_t workspace_floats, hipStream_t stream);
size_t latent_attention_workspace_floats(int kv_rank);
// out[t, h*value_dim + e] = sum_r w_uv[h*value_dim + e, r] * o_lat[t, h, r]
void latent_expand(const Tensor2& o_lat, const Tensor2& w_uv, const Tensor2& out, const LatentShape& sh, hipStream_t stream);

// -- attention with shaped scores -------------------------------------------------------------------
// out = in + conv(in): a causal convolution per channel over `taps` inputs (taps [channels, taps], the last tap
// the token's own), added onto its input; in fp32 [T, C], out in its own dtype. Carried inputs as for conv_silu.
// With `residual` false the input is not added: out = conv(in) alone.
void conv_residual(const Tensor2& in, const Tensor2& weight, const StateArgs& st, const Tensor2& out, hipStream_t stream, bool residual = true);
// The same behind an RMS norm, in one kernel, for a step in which every sequence brings one token (x.rows == st.n_seqs):
// out = h + conv(h) with h = x / sqrt(mean(x^2) + eps) * norm_weight.
// False (and nothing done): sizes the kernel is not made for (more than 8 taps, rows wider than 2,048).
bool rmsnorm_conv_single(const Tensor2& x, const float* norm_weight, float eps, const Tensor2& weight, const StateArgs& st,
                         const Tensor2& out, hipStream_t stream);
// For the same kind of step, a convolution that reads the stream itself: out = x + conv(x); and, with `y` (a sub-layer's
// result, fp32, x's shape) and a norm's weight, behind x += y / sqrt(mean(y^2) + eps) * norm_weight (x is written) in
// the same kernel. False (and nothing done): sizes the kernel is not made for, as above.
bool stream_conv_single(const Tensor2& x, const Tensor2* y, const float* norm_weight, float eps, const Tensor2& weight,
                        const StateArgs& st, const Tensor2& out, hipStream_t stream);
// x += mult * sum_k rmsnorm(y_k) * w_k: n inputs of x's shape one behind the other in `ys` ([n * rows, size] fp32), their
// weights one behind the other in `weights` ([n * size]); 2 to 4 inputs, rows of up to 2,048 columns.
void rmsnorm_add_many(const Tensor2& ys, const float* weights, int n, float mult, float eps, const Tensor2& x, hipStream_t stream);
// Sizes and constants of an attention whose scores are shaped before the softmax (kernels/scored_attention.hip).
struct ScoredShape {
    int n_heads = 0, n_kv_heads = 0, dim = 0, value_dim = 0;
    float scale = 1.f, softcap = 0.f;          // softcap <= 0: none
    int window = 0, chunk = 0;                 // sliding window or chunked causal mask; both 0: plain causal
    const float* r1 = nullptr;                 // per head: s -= r1 ln(1 + r2 (i - j)); null: none
    const float* r2 = nullptr;
    int keep_first = 0;                        // with a window: the sequence's first keep_first positions stay visible too
    const float* slope = nullptr;              // per head: s -= slope (i - j) (instead of r1, r2); null: none
    const float* sink = nullptr;               // per head: one more term exp(sink) in the softmax's denominator; null: none
    int norm_mode = 0;                         // 0 none, 1 per head with one weight [dim], 2 over the whole row,
                                               // 3 every head to unit root mean square BEHIND the rotation, no weight
    const float* q_norm = nullptr;
    const float* k_norm = nullptr;
    float eps = 1e-6f;
    int rot_dims = 0;                          // the first rot_dims columns of a head are turned (half-split pairs,
    bool rot_interleaved = false;              // or with rot_interleaved column 2i with column 2i + 1)
    double rot_base = 10000.0;
    // weights without a softmax: a visible key's weight is sigmoid(score + score_bias[h]) (score_bias per head, or
    // null), not normalised over the keys
    bool sigmoid_weights = false;
    const float* score_bias = nullptr;
    bool gate_per_head = false;                // the gate has one column per head instead of one per value column
};
// From the fp32 rows of the input projection (queries at q_col, keys at k_col, values at v_col; v_col < 0: the
// values are the keys before their norm): q [T, heads * dim] normed and turned, and the keys and values written
// to their page rows (slots[t]). k_col < 0: queries only (the keys and values are another layer's; the pages are
// not touched and may be empty tensors).
void qk_prepare(const Tensor2& proj, int q_col, int k_col, int v_col, const ScoredShape& sh, const int* positions,
                const int* slots, const Tensor2& q, const Tensor2& k_pages, const Tensor2& v_pages, hipStream_t stream);
struct ScoredStep {
    const int* block_tables = nullptr;     // [n_seqs, max_blocks]
    int max_blocks = 0, n_seqs = 0, max_q_len = 0, max_ctx_len = 0, page_size = 0;
    int n_single = 0;                      // the first n_single sequences bring one token each
    const int* token_seq = nullptr;        // [T]
    const int* positions = nullptr;        // [T]
    const int* cu_q = nullptr;             // [n_seqs + 1]
    const int* ctx_len = nullptr;          // [n_seqs]
};
// out[t, h] = sum_j softmax_j(shaped score) v_j over the visible keys of the pages, times sigmoid(gate[t, gate_col +
// h * value_dim ..]) if a gate (fp32 rows) is given.
void scored_attention(const Tensor2& q, const Tensor2& k_pages, const Tensor2& v_pages, const ScoredStep& step,
                      const ScoredShape& sh, const Tensor2* gate, int gate_col, const Tensor2& out, hipStream_t stream);

// -- gated linear recurrence (HGRN2) ----------------------------------------------------------------
// proj (fp32 rows): raw queries at q_col and raw gates at f_col (heads * dim each), values at v_col (heads * value_dim).
// y: hgrn2_parts(dim) shares [T, heads * value_dim], y.rows * y.stride floats apart; the state ([heads][dim][value_dim]
// fp32) lies state_offset floats into a request's slot.
// Portions longer than hgrn2_chunk() tokens are cut into chunks that run side by side, for which `workspace`
// (hgrn2_workspace_floats floats) is needed; without it they run token by token.
void hgrn2_scan(const Tensor2& proj, int q_col, int f_col, int v_col, const float* f_bias, const float* lower, const StateArgs& st,
                size_t state_offset, int heads, int dim, int value_dim, const Tensor2& y, float* workspace, size_t workspace_floats,
                hipStream_t stream);
int hgrn2_parts(int dim);
int hgrn2_chunk();
size_t hgrn2_workspace_floats(int tokens, int n_seqs, int heads, int dim, int value_dim);
// -- linear attention with a decay ------------------------------------------------------------------
// Per head S <- diag(f) S + k v^T, o = S^T q with q = q_scale * proj[q_col..], k = k_scale * proj[k_col..] (heads * dim
// each) and v = proj[v_col..] (heads * value_dim) from proj's fp32 rows. The decays f come per token and channel from
// `decay` ([T, heads * dim] fp32) or, if that is null, one per head from `head_decay` ([heads] fp32, on the device).
// Shares of y, state, chunks and workspace as for hgrn2_scan (the same kernels; hgrn2_parts, hgrn2_chunk and
// hgrn2_workspace_floats give the sizes).
void decay_scan(const Tensor2& proj, int q_col, int k_col, int v_col, const Tensor2* decay, const float* head_decay, float q_scale,
                float k_scale, const StateArgs& st, size_t state_offset, int heads, int dim, int value_dim, const Tensor2& y,
                float* workspace, size_t workspace_floats, hipStream_t stream);
// The first rot_dims columns of n_heads heads of `dim` columns, from column col0 of proj's fp32 rows, turned in place by
// the tokens' positions (column i pairs with i + rot_dims / 2, angle p * base^(-2i / rot_dims)).
void rotary_rows(const Tensor2& proj, int col0, int n_heads, int dim, int rot_dims, double base, const int* positions, hipStream_t stream);
// out[t, c] = sigmoid(w[c, :] . proj[t, a_col : a_col + rank] + bias[c])^(1 / tau): w [N, rank] fp32, out [T, N] fp32.
void lowrank_decay(const Tensor2& proj, int a_col, const Tensor2& w, const float* bias, float tau, const Tensor2& out, hipStream_t stream);
// out = rmsnorm(x) * weight * silu(gate[:, gate_col ..]) in `groups` equal parts of the columns, the gate BEHIND the norm
// (weight [x.cols] or null; gate fp32 rows). Parts as for rmsnorm.
void rmsnorm_gate_after(const Tensor2& x, const float* weight, float eps, int groups, const Tensor2& gate, int gate_col, const Tensor2& out,
                        hipStream_t stream, int parts = 1, size_t part_stride = 0);
// x <- cap tanh(x / cap) (contiguous fp32)
void softcap(const Tensor2& x, float cap, hipStream_t stream);
// `kept` holds n_old earlier streams of x's shape one behind the other ([>= (n_old + 1) * rows, cols] fp32, contiguous).
// x is stored behind them as stream n_old, and x <- sum_(j <= n_old) w[j] stream_j (w: n_old + 1 floats on the device).
void depth_mix(const Tensor2& x, const Tensor2& kept, int n_old, const float* w, hipStream_t stream);

// -- mixture of experts -----------------------------------------------------------------------------
// From a token's router logits ([T, E] fp32): scores softmax(logits) over all experts, the `top` largest chosen (the
// lower index wins a tie), weight_e = scale * score_e for them and 0 for the others. Then
// out[t, e * ff + j] = weight_e * relu(up[t, e * ff + j])^2 for the E experts of ff columns; the columns behind them (a
// shared expert's) are relu(.)^2 alone. out may be up. `weights` (optional, [T, E] fp32) receives the weights.
void moe_act(const Tensor2& up, const Tensor2& logits, int ff, int top, float scale, const Tensor2& out, const Tensor2* weights,
             hipStream_t stream);
// The routed experts' activation for gated, clamped experts (kernels/moe.hip): up [T, 2 (E ff + shared_ff)] with rows
// [expert: gate | up] ... [shared: gate | up], logits [T, E (+ 1: the shared expert's gate)] fp32, out [T, E ff + shared_ff].
struct MoeGlu {
    int experts = 0, ff = 0, shared_ff = 0, top = 0;
    float scale = 1.f, limit = 0.f, shared_limit = 0.f, alpha = 1.f;
    bool sigmoid_router = false, weight_on_input = false, shared_gate = false;
};
void moe_glu_act(const Tensor2& up, const Tensor2& logits, const MoeGlu& m, const Tensor2& out, hipStream_t stream);

// out = [a | b] row by row in out's dtype (a, b fp32 [T, D])
void concat_cast(const Tensor2& a, const Tensor2& b, const Tensor2& out, hipStream_t stream);
// out[t, j] = act(gu[t, j]) * gu[t, F + j] (act: GELU_TANH or GLU_SILU)
void glu_act(const Tensor2& gu, int act, const Tensor2& out, hipStream_t stream);

// `mirror` (optional): a second place for the chosen tokens, which may be pinned host memory (the kernel that
// chooses writes it: no copy has to be launched for the host to read them).
void argmax(const Tensor2& logits, int* out, hipStream_t stream, int* mirror = nullptr);
void sample(const Tensor2& logits, const float* temperature, const float* u, int* out, hipStream_t stream, int* mirror = nullptr);

}  // namespace minillm
