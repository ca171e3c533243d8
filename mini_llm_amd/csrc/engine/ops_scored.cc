// Checked dispatch of the attention with shaped scores, the gated linear recurrence, the convolution added
// onto its input and their small companions (declared in ops.h beside the other ops).
#include <algorithm>

#include "kernels.h"
#include "ops.h"

namespace minillm {

namespace {
void check(int rc, const char* what) {
    if (rc == 0) return;
    if (rc < 0) fail("%s: the kernel refuses these sizes (code %d)", what, rc);
    fail("%s: HIP error %d (%s) at launch", what, rc, hipGetErrorString(static_cast<hipError_t>(rc)));
}
void need_act(const Tensor2& t, const char* name) {
    if (t.dtype != F32 && t.dtype != BF16) fail("%s: unsupported dtype code %d (float32 or bfloat16)", name, t.dtype);
    if (t.data == nullptr && t.rows * t.cols > 0) fail("%s: null data pointer", name);
}
void need_f32(const Tensor2& t, const char* name) {
    if (t.dtype != F32 || (t.data == nullptr && t.rows * t.cols > 0)) fail("%s must be float32", name);
}
int i32(int64_t v) { return static_cast<int>(v); }

void check_state(const StateArgs& st, size_t floats_needed, const char* what) {
    if (st.token_seq == nullptr || st.cu_q == nullptr || st.state_slots == nullptr || st.n_seqs < 1)
        fail("%s: the step's token_seq, cu_q and state slots are needed", what);
    if (st.state == nullptr || st.n_slots < 1 || st.slot_floats < floats_needed)
        fail("%s: a state slot holds %zu floats, %zu are needed", what, st.slot_floats, floats_needed);
}

void check_shape(const ScoredShape& sh, const char* what) {
    if (sh.n_heads < 1 || sh.n_kv_heads < 1 || sh.n_heads % sh.n_kv_heads != 0 || sh.dim < 1 || sh.value_dim < 1)
        fail("%s: %d heads over %d key/value heads of %d / %d do not fit", what, sh.n_heads, sh.n_kv_heads, sh.dim, sh.value_dim);
    if (sh.window < 0 || sh.chunk < 0 || (sh.window > 0 && sh.chunk > 0)) fail("%s: a window or a chunk, not both", what);
    if ((sh.r1 != nullptr) != (sh.r2 != nullptr)) fail("%s: the distance bias needs both of its numbers per head", what);
    if (sh.slope != nullptr && sh.r1 != nullptr) fail("%s: a linear or a logarithmic distance bias, not both", what);
    if (sh.sink != nullptr && sh.sigmoid_weights) fail("%s: a sink stands in a softmax's denominator; sigmoid weights have none", what);
    if (sh.keep_first < 0 || (sh.keep_first > 0 && sh.window <= 0)) fail("%s: kept first positions go with a sliding window", what);
}
}  // namespace

void conv_residual(const Tensor2& in, const Tensor2& weight, const StateArgs& st, const Tensor2& out, hipStream_t stream, bool residual) {
    need_f32(in, "conv_residual: the input");
    need_f32(weight, "conv_residual: the taps");
    need_act(out, "conv_residual: out");
    const int C = i32(weight.rows), taps = i32(weight.cols);
    if (!weight.contiguous() || taps < 1 || taps > 16) fail("conv_residual: taps [channels, 1 to 16] contiguous are needed");
    if (in.cols != C || out.cols != C || out.rows != in.rows) fail("conv_residual: input and out must be [T, %d]", C);
    // (a single tap reads no carried rows: such a convolution needs no state, only the step's arrays)
    if (taps > 1) check_state(st, static_cast<size_t>(taps - 1) * C, "conv_residual");
    else if (st.token_seq == nullptr || st.cu_q == nullptr || st.state_slots == nullptr || st.n_seqs < 1)
        fail("conv_residual: the step's token_seq, cu_q and state slots are needed");
    check(mllm_conv_residual(static_cast<const float*>(in.data), i32(in.stride), C, static_cast<const float*>(weight.data), taps, st.token_seq,
                             st.cu_q, st.state_slots, st.state, st.slot_floats, out.data, i32(out.stride), out.dtype, i32(in.rows), st.n_seqs,
                             st.write ? 1 : 0, stream, residual ? 1 : 0), "conv_residual");
}

bool rmsnorm_conv_single(const Tensor2& x, const float* norm_weight, float eps, const Tensor2& weight, const StateArgs& st,
                         const Tensor2& out, hipStream_t stream) {
    need_f32(x, "rmsnorm_conv_single: the input");
    need_f32(weight, "rmsnorm_conv_single: the taps");
    need_act(out, "rmsnorm_conv_single: out");
    const int C = i32(weight.rows), taps = i32(weight.cols);
    if (!weight.contiguous() || taps < 1 || taps > 16 || norm_weight == nullptr) fail("rmsnorm_conv_single: taps [channels, 1 to 16] contiguous and the norm's weight are needed");
    if (x.cols != C || out.cols != C || out.rows != x.rows) fail("rmsnorm_conv_single: input and out must be [T, %d]", C);
    if (x.rows != st.n_seqs || st.state_slots == nullptr) fail("rmsnorm_conv_single: every sequence of the step must bring one token");
    if (taps > 1 && (st.state == nullptr || st.slot_floats < static_cast<size_t>(taps - 1) * C))
        fail("rmsnorm_conv_single: a state slot holds %zu floats, %zu are needed", st.slot_floats, static_cast<size_t>(taps - 1) * C);
    const int rc = mllm_rmsnorm_conv_single(static_cast<const float*>(x.data), i32(x.stride), norm_weight, eps, C, static_cast<const float*>(weight.data), taps,
                                            st.state_slots, st.state, st.slot_floats, out.data, i32(out.stride), out.dtype, i32(x.rows), st.write ? 1 : 0, stream);
    if (rc == -2) return false;
    check(rc, "rmsnorm_conv_single");
    return true;
}

bool stream_conv_single(const Tensor2& x, const Tensor2* y, const float* norm_weight, float eps, const Tensor2& weight,
                        const StateArgs& st, const Tensor2& out, hipStream_t stream) {
    need_f32(x, "stream_conv_single: the stream");
    need_f32(weight, "stream_conv_single: the taps");
    need_act(out, "stream_conv_single: out");
    const int C = i32(weight.rows), taps = i32(weight.cols);
    if (!weight.contiguous() || taps < 1 || taps > 16) fail("stream_conv_single: taps [channels, 1 to 16] contiguous are needed");
    if (x.cols != C || out.cols != C || out.rows != x.rows) fail("stream_conv_single: stream and out must be [T, %d]", C);
    if (y != nullptr) {
        need_f32(*y, "stream_conv_single: the sub-layer's result");
        if (y->rows != x.rows || y->cols != C || norm_weight == nullptr) fail("stream_conv_single: the result must be [T, %d] and comes with a norm's weight", C);
    }
    if (x.rows != st.n_seqs || st.state_slots == nullptr) fail("stream_conv_single: every sequence of the step must bring one token");
    if (taps > 1 && (st.state == nullptr || st.slot_floats < static_cast<size_t>(taps - 1) * C))
        fail("stream_conv_single: a state slot holds %zu floats, %zu are needed", st.slot_floats, static_cast<size_t>(taps - 1) * C);
    const int rc = mllm_stream_conv_single(static_cast<float*>(x.data), i32(x.stride), y ? static_cast<const float*>(y->data) : nullptr,
                                           y ? i32(y->stride) : 0, y ? norm_weight : nullptr, eps, C, static_cast<const float*>(weight.data), taps,
                                           st.state_slots, st.state, st.slot_floats, out.data, i32(out.stride), out.dtype, i32(x.rows),
                                           st.write ? 1 : 0, stream);
    if (rc == -2) return false;
    check(rc, "stream_conv_single");
    return true;
}

void rmsnorm_add_many(const Tensor2& ys, const float* weights, int n, float mult, float eps, const Tensor2& x, hipStream_t stream) {
    need_f32(ys, "rmsnorm_add_many: the inputs");
    need_f32(x, "rmsnorm_add_many: x");
    if (n < 2 || n > 4 || weights == nullptr || x.cols > 2048) fail("rmsnorm_add_many: two to four inputs with their weights, rows of up to 2,048 columns");
    if (!ys.contiguous() || !x.contiguous() || ys.rows != x.rows * n || ys.cols != x.cols) fail("rmsnorm_add_many: the inputs must be [%d * rows, size] beside x [rows, size]", n);
    check(mllm_rmsnorm_add_many(static_cast<const float*>(ys.data), static_cast<size_t>(x.rows) * x.cols, weights, static_cast<size_t>(x.cols), n, mult, eps,
                                static_cast<float*>(x.data), i32(x.rows), i32(x.cols), stream), "rmsnorm_add_many");
}

void qk_prepare(const Tensor2& proj, int q_col, int k_col, int v_col, const ScoredShape& sh, const int* positions,
                const int* slots, const Tensor2& q, const Tensor2& k_pages, const Tensor2& v_pages, hipStream_t stream) {
    check_shape(sh, "qk_prepare");
    need_f32(proj, "qk_prepare: the projection");
    need_act(q, "qk_prepare: q");
    const int64_t nq = static_cast<int64_t>(sh.n_heads) * sh.dim, nk = static_cast<int64_t>(sh.n_kv_heads) * sh.dim,
                  nv = static_cast<int64_t>(sh.n_kv_heads) * sh.value_dim;
    const bool keys = k_col >= 0;
    if (q_col < 0 || q_col + nq > proj.cols || (keys && k_col + nk > proj.cols) || (keys && v_col >= 0 && v_col + nv > proj.cols))
        fail("qk_prepare: queries, keys or values lie outside the projection's rows of %lld", (long long)proj.cols);
    if (keys && v_col < 0 && sh.value_dim != sh.dim) fail("qk_prepare: values taken from the keys must have the keys' width");
    if (q.rows != proj.rows || q.cols != nq) fail("qk_prepare: q must be [T, %lld]", (long long)nq);
    if (!keys) {
        if (sh.norm_mode == 2) fail("qk_prepare: a norm over the whole row needs the keys");
        check(mllm_qk_prepare(static_cast<const float*>(proj.data), i32(proj.stride), q_col, 0, 0, i32(proj.rows), sh.n_heads, 0,
                              sh.dim, sh.value_dim, sh.norm_mode, sh.q_norm, sh.q_norm, sh.eps, sh.rot_dims, sh.rot_base, positions, nullptr, q.data,
                              i32(q.stride), nullptr, nullptr, q.dtype, stream, sh.rot_interleaved ? 1 : 0), "qk_prepare");
        return;
    }
    if (k_pages.dtype != q.dtype || v_pages.dtype != q.dtype || !k_pages.contiguous() || !v_pages.contiguous() || k_pages.cols != nk ||
        v_pages.cols != nv || k_pages.rows != v_pages.rows)
        fail("qk_prepare: the pages must be contiguous [rows, %lld] and [rows, %lld] %s", (long long)nk, (long long)nv, dtype_name(q.dtype));
    if (positions == nullptr || slots == nullptr) fail("qk_prepare: positions and page rows are needed");
    if (sh.norm_mode < 0 || sh.norm_mode > 3 || ((sh.norm_mode == 1 || sh.norm_mode == 2) && (sh.q_norm == nullptr || sh.k_norm == nullptr)))
        fail("qk_prepare: norm mode %d needs its two weights", sh.norm_mode);
    if (sh.rot_dims < 0 || sh.rot_dims % 2 != 0 || sh.rot_dims > sh.dim || (sh.rot_dims > 0 && !(sh.rot_base > 0)))
        fail("qk_prepare: %d turned columns of %d (even, at most the head) and a positive base are needed", sh.rot_dims, sh.dim);
    check(mllm_qk_prepare(static_cast<const float*>(proj.data), i32(proj.stride), q_col, k_col, v_col, i32(proj.rows), sh.n_heads, sh.n_kv_heads,
                          sh.dim, sh.value_dim, sh.norm_mode, sh.q_norm, sh.k_norm, sh.eps, sh.rot_dims, sh.rot_base, positions, slots, q.data,
                          i32(q.stride), k_pages.data, v_pages.data, q.dtype, stream, sh.rot_interleaved ? 1 : 0), "qk_prepare");
}

void scored_attention(const Tensor2& q, const Tensor2& k_pages, const Tensor2& v_pages, const ScoredStep& step,
                      const ScoredShape& sh, const Tensor2* gate, int gate_col, const Tensor2& out, hipStream_t stream) {
    check_shape(sh, "scored_attention");
    need_act(q, "scored_attention: q");
    const int64_t nq = static_cast<int64_t>(sh.n_heads) * sh.dim, nk = static_cast<int64_t>(sh.n_kv_heads) * sh.dim,
                  nv = static_cast<int64_t>(sh.n_kv_heads) * sh.value_dim, no = static_cast<int64_t>(sh.n_heads) * sh.value_dim;
    if (q.cols != nq) fail("scored_attention: q must be [T, %lld]", (long long)nq);
    if (out.dtype != q.dtype || out.rows != q.rows || out.cols != no) fail("scored_attention: out must be [T, %lld] %s", (long long)no, dtype_name(q.dtype));
    if (k_pages.dtype != q.dtype || v_pages.dtype != q.dtype || !k_pages.contiguous() || !v_pages.contiguous() || k_pages.cols != nk ||
        v_pages.cols != nv || k_pages.rows != v_pages.rows)
        fail("scored_attention: the pages must be contiguous [rows, %lld] and [rows, %lld] %s", (long long)nk, (long long)nv, dtype_name(q.dtype));
    if (step.page_size < 1 || k_pages.rows % step.page_size != 0) fail("scored_attention: the page pool is not a whole number of pages");
    if (step.block_tables == nullptr || step.token_seq == nullptr || step.positions == nullptr || step.max_blocks < 1)
        fail("scored_attention: block tables, token_seq and positions are needed");
    const float* g = nullptr;
    int ldg = 0;
    if (gate != nullptr) {
        need_f32(*gate, "scored_attention: the gate");
        if (gate->rows != q.rows || gate_col < 0 || gate_col + (sh.gate_per_head ? sh.n_heads : no) > gate->cols) fail("scored_attention: the gate's columns lie outside its rows");
        g = static_cast<const float*>(gate->data) + gate_col;
        ldg = i32(gate->stride);
    }
    // keys and values of one width: the kernels that every attention of the engine runs on (tiles of queries for
    // prompt portions, split keys for single tokens), with the shaping handed on; they fall back by themselves to
    // the one-wavefront-per-row kernel below for sizes they do not take
    // (sigmoid weights: the matrix-core tiles and the split-key kernel in bfloat16 at their head sizes; 32-bit and
    // other sizes stay with the kernel below)
    const bool special = sh.sigmoid_weights;
    const bool special_ok = q.dtype == BF16 && (sh.dim == 32 || sh.dim == 64 || sh.dim == 128) && step.page_size >= sh.dim / 16 &&
                            (step.page_size & (step.page_size - 1)) == 0 && step.max_blocks <= 2048;
    if (tuning().scored_shared_kernels && (!special || special_ok) && sh.dim == sh.value_dim && sh.dim % 8 == 0 && sh.dim <= 256 && (q.stride * q.esz()) % 16 == 0 && (sh.dim * q.esz()) % 16 == 0 &&
        (reinterpret_cast<uintptr_t>(q.data) & 15) == 0 && (g == nullptr || sh.gate_per_head || (ldg % 4 == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0)) &&
        (reinterpret_cast<uintptr_t>(out.data) & 15) == 0 && (out.stride * out.esz()) % 8 == 0 &&
        step.cu_q != nullptr && step.ctx_len != nullptr && step.n_seqs > 0) {
        const MllmScoreShape shape{sh.softcap, sh.chunk, sh.r1, sh.r2, sh.sigmoid_weights ? 1 : 0, sh.score_bias, sh.gate_per_head ? 1 : 0,
                                   sh.slope, sh.sink, sh.keep_first};
        AttentionArgs a;
        a.q = q; a.q_col = 0; a.n_heads = sh.n_heads; a.n_kv_heads = sh.n_kv_heads; a.head_dim = sh.dim;
        a.k_pages = k_pages; a.v_pages = v_pages; a.page_size = step.page_size;
        a.block_tables = step.block_tables; a.n_seqs = step.n_seqs; a.max_blocks = step.max_blocks;
        a.token_seq = step.token_seq; a.positions = step.positions; a.scale = sh.scale; a.window = sh.window;
        a.out = out; a.cu_q = step.cu_q; a.ctx_len = step.ctx_len; a.max_q_len = step.max_q_len; a.max_ctx_len = step.max_ctx_len;
        a.n_single = step.n_single; a.shape = &shape; a.gate = g; a.gate_stride = ldg;
        paged_attention(a, nullptr, stream);
        return;
    }
    check(mllm_scored_attention_rows(q.data, i32(q.stride), k_pages.data, v_pages.data, step.block_tables, step.max_blocks, step.token_seq,
                                     step.positions, i32(q.rows), sh.n_heads, sh.n_kv_heads, sh.dim, sh.value_dim, step.page_size, sh.scale,
                                     sh.softcap, sh.window, sh.chunk, sh.r1, sh.r2, g, ldg, out.data, i32(out.stride), q.dtype, stream,
                                     sh.sigmoid_weights ? 1 : 0, sh.score_bias, sh.gate_per_head ? 1 : 0, sh.slope, sh.sink, sh.keep_first),
          "scored_attention");
}

int hgrn2_parts(int dim) { return mllm_hgrn2_parts(dim); }
int hgrn2_chunk() { return mllm_hgrn2_chunk(); }
size_t hgrn2_workspace_floats(int tokens, int n_seqs, int heads, int dim, int value_dim) {
    return mllm_hgrn2_workspace_floats(tokens, n_seqs, heads, dim, value_dim);
}

void hgrn2_scan(const Tensor2& proj, int q_col, int f_col, int v_col, const float* f_bias, const float* lower, const StateArgs& st,
                size_t state_offset, int heads, int dim, int value_dim, const Tensor2& y, float* workspace, size_t workspace_floats,
                hipStream_t stream) {
    need_f32(proj, "hgrn2_scan: the projection");
    need_f32(y, "hgrn2_scan: y");
    if (heads < 1 || dim < 1 || value_dim < 1) fail("hgrn2_scan: heads and sizes must be positive");
    const int64_t nq = static_cast<int64_t>(heads) * dim, nv = static_cast<int64_t>(heads) * value_dim;
    if (q_col < 0 || q_col + nq > proj.cols || f_col < 0 || f_col + nq > proj.cols || v_col < 0 || v_col + nv > proj.cols)
        fail("hgrn2_scan: queries, gates or values lie outside the projection's rows of %lld", (long long)proj.cols);
    if (y.rows != proj.rows || y.cols != nv) fail("hgrn2_scan: y must be [%lld, %lld]", (long long)proj.rows, (long long)nv);
    if (lower == nullptr) fail("hgrn2_scan: the gates' lower bounds are needed");
    check_state(st, state_offset + static_cast<size_t>(heads) * dim * value_dim, "hgrn2_scan");
    const int T = i32(proj.rows);
    // (a step whose longest portion is unknown is taken to have a long one)
    const int max_q = st.max_q_len > 0 ? st.max_q_len : T;
    if (workspace != nullptr && workspace_floats < hgrn2_workspace_floats(T, st.n_seqs, heads, dim, value_dim))
        fail("hgrn2_scan: the workspace holds %zu floats, %zu are needed", workspace_floats, hgrn2_workspace_floats(T, st.n_seqs, heads, dim, value_dim));
    check(mllm_hgrn2_scan(static_cast<const float*>(proj.data), i32(proj.stride), q_col, f_col, v_col, f_bias, lower, st.cu_q, st.state_slots,
                          st.state, st.slot_floats, state_offset, static_cast<float*>(y.data), i32(y.stride), static_cast<size_t>(y.rows) * y.stride,
                          T, st.n_seqs, max_q, heads, dim, value_dim, st.write ? 1 : 0, workspace, stream), "hgrn2_scan");
}

void decay_scan(const Tensor2& proj, int q_col, int k_col, int v_col, const Tensor2* decay, const float* head_decay, float q_scale,
                float k_scale, const StateArgs& st, size_t state_offset, int heads, int dim, int value_dim, const Tensor2& y,
                float* workspace, size_t workspace_floats, hipStream_t stream) {
    need_f32(proj, "decay_scan: the projection");
    need_f32(y, "decay_scan: y");
    if (heads < 1 || dim < 1 || value_dim < 1) fail("decay_scan: heads and sizes must be positive");
    const int64_t nq = static_cast<int64_t>(heads) * dim, nv = static_cast<int64_t>(heads) * value_dim;
    if (q_col < 0 || q_col + nq > proj.cols || k_col < 0 || k_col + nq > proj.cols || v_col < 0 || v_col + nv > proj.cols)
        fail("decay_scan: queries, keys or values lie outside the projection's rows of %lld", (long long)proj.cols);
    if (y.rows != proj.rows || y.cols != nv) fail("decay_scan: y must be [%lld, %lld]", (long long)proj.rows, (long long)nv);
    if (decay != nullptr) {
        need_f32(*decay, "decay_scan: the decays");
        if (decay->rows != proj.rows || decay->cols != nq) fail("decay_scan: the decays must be [%lld, %lld]", (long long)proj.rows, (long long)nq);
    } else if (head_decay == nullptr) {
        fail("decay_scan: decays per token and channel, or one per head, are needed");
    }
    check_state(st, state_offset + static_cast<size_t>(heads) * dim * value_dim, "decay_scan");
    const int T = i32(proj.rows);
    const int max_q = st.max_q_len > 0 ? st.max_q_len : T;
    if (workspace != nullptr && workspace_floats < hgrn2_workspace_floats(T, st.n_seqs, heads, dim, value_dim))
        fail("decay_scan: the workspace holds %zu floats, %zu are needed", workspace_floats, hgrn2_workspace_floats(T, st.n_seqs, heads, dim, value_dim));
    check(mllm_decay_scan(static_cast<const float*>(proj.data), i32(proj.stride), q_col, k_col, v_col, decay ? static_cast<const float*>(decay->data) : nullptr,
                          decay ? i32(decay->stride) : 0, head_decay, q_scale, k_scale, st.cu_q, st.state_slots, st.state, st.slot_floats, state_offset,
                          static_cast<float*>(y.data), i32(y.stride), static_cast<size_t>(y.rows) * y.stride, T, st.n_seqs, max_q, heads, dim, value_dim,
                          st.write ? 1 : 0, workspace, stream), "decay_scan");
}

void rotary_rows(const Tensor2& proj, int col0, int n_heads, int dim, int rot_dims, double base, const int* positions, hipStream_t stream) {
    need_f32(proj, "rotary_rows: the projection");
    if (n_heads < 1 || dim < 1 || col0 < 0 || col0 + static_cast<int64_t>(n_heads) * dim > proj.cols) fail("rotary_rows: the heads lie outside the projection's rows");
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > dim || (rot_dims > 0 && !(base > 0))) fail("rotary_rows: %d turned columns of %d (even, at most the head) and a positive base are needed", rot_dims, dim);
    if (positions == nullptr) fail("rotary_rows: positions are needed");
    check(mllm_rotary_rows(static_cast<float*>(proj.data), i32(proj.stride), col0, i32(proj.rows), n_heads, dim, rot_dims, base, positions, stream), "rotary_rows");
}

void lowrank_decay(const Tensor2& proj, int a_col, const Tensor2& w, const float* bias, float tau, const Tensor2& out, hipStream_t stream) {
    need_f32(proj, "lowrank_decay: the projection");
    need_f32(w, "lowrank_decay: the map");
    need_f32(out, "lowrank_decay: out");
    if (!w.contiguous() || w.cols < 1 || a_col < 0 || a_col + w.cols > proj.cols) fail("lowrank_decay: the low-rank values lie outside the projection's rows");
    if (out.rows != proj.rows || out.cols != w.rows) fail("lowrank_decay: out must be [%lld, %lld]", (long long)proj.rows, (long long)w.rows);
    if (!(tau > 0.f)) fail("lowrank_decay: tau must be positive");
    check(mllm_lowrank_decay(static_cast<const float*>(proj.data), i32(proj.stride), a_col, i32(w.cols), static_cast<const float*>(w.data), bias, tau,
                             static_cast<float*>(out.data), i32(out.stride), i32(proj.rows), i32(w.rows), stream), "lowrank_decay");
}

void rmsnorm_gate_after(const Tensor2& x, const float* weight, float eps, int groups, const Tensor2& gate, int gate_col, const Tensor2& out,
                        hipStream_t stream, int parts, size_t part_stride) {
    need_f32(x, "rmsnorm_gate_after: x");
    need_f32(gate, "rmsnorm_gate_after: the gate");
    need_act(out, "rmsnorm_gate_after: out");
    if (groups < 1 || x.cols % groups != 0) fail("rmsnorm_gate_after: %lld columns in %d groups", (long long)x.cols, groups);
    if (out.rows != x.rows || out.cols != x.cols || gate.rows != x.rows || gate_col < 0 || gate_col + x.cols > gate.cols)
        fail("rmsnorm_gate_after: out and the gate's columns must match x [%lld, %lld]", (long long)x.rows, (long long)x.cols);
    check(mllm_rmsnorm_gate_after(static_cast<const float*>(x.data), i32(x.stride), weight, static_cast<const float*>(gate.data) + gate_col, i32(gate.stride),
                                  out.data, i32(out.stride), i32(x.rows), i32(x.cols), groups, eps, out.dtype, parts, part_stride, stream), "rmsnorm_gate_after");
}

void softcap(const Tensor2& x, float cap, hipStream_t stream) {
    need_f32(x, "softcap: x");
    if (!x.contiguous()) fail("softcap: x must be contiguous");
    if (!(cap > 0.f)) fail("softcap: the cap must be positive");
    check(mllm_softcap(static_cast<float*>(x.data), static_cast<size_t>(x.rows) * x.cols, cap, stream), "softcap");
}

void depth_mix(const Tensor2& x, const Tensor2& kept, int n_old, const float* w, hipStream_t stream) {
    need_f32(x, "depth_mix: x");
    need_f32(kept, "depth_mix: the kept streams");
    if (!x.contiguous() || !kept.contiguous() || kept.cols != x.cols || n_old < 0 || kept.rows < x.rows * (n_old + 1))
        fail("depth_mix: %d kept streams and the new one do not fit [%lld, %lld]", n_old, (long long)kept.rows, (long long)kept.cols);
    if (w == nullptr) fail("depth_mix: the weights are missing");
    check(mllm_depth_mix(static_cast<float*>(x.data), static_cast<float*>(kept.data), static_cast<size_t>(x.rows) * x.cols, n_old, w,
                         static_cast<size_t>(x.rows) * x.cols, stream), "depth_mix");
}

void moe_act(const Tensor2& up, const Tensor2& logits, int ff, int top, float scale, const Tensor2& out, const Tensor2* weights,
             hipStream_t stream) {
    need_act(up, "moe_act: up");
    need_f32(logits, "moe_act: the router's logits");
    if (out.dtype != up.dtype || out.rows != up.rows || out.cols != up.cols) fail("moe_act: out must have up's shape and dtype");
    const int E = i32(logits.cols);
    if (logits.rows != up.rows || E < 1 || ff < 1 || static_cast<int64_t>(E) * ff > up.cols) fail("moe_act: %d experts of %d columns do not fit rows of %lld", E, ff, (long long)up.cols);
    if (top < 1 || top > E) fail("moe_act: %d of %d experts", top, E);
    float* wp = nullptr;
    int ldw = 0;
    if (weights != nullptr) {
        need_f32(*weights, "moe_act: the weights");
        if (weights->rows != up.rows || weights->cols != E) fail("moe_act: the weights must be [%lld, %d]", (long long)up.rows, E);
        wp = static_cast<float*>(weights->data);
        ldw = i32(weights->stride);
    }
    check(mllm_moe_act(up.data, i32(up.stride), static_cast<const float*>(logits.data), i32(logits.stride), E, ff, i32(up.cols) - E * ff, top, scale,
                       out.data, i32(out.stride), wp, ldw, i32(up.rows), up.dtype, stream), "moe_act");
}

void moe_glu_act(const Tensor2& up, const Tensor2& logits, const MoeGlu& m, const Tensor2& out, hipStream_t stream) {
    need_act(up, "moe_glu_act: up");
    need_f32(logits, "moe_glu_act: the router's logits");
    const int64_t n = static_cast<int64_t>(m.experts) * m.ff + m.shared_ff;
    if (m.experts < 1 || m.ff < 1 || m.shared_ff < 0 || m.top < 1 || m.top > m.experts) fail("moe_glu_act: %d of %d experts of %d do not fit", m.top, m.experts, m.ff);
    if (out.dtype != up.dtype || out.rows != up.rows || out.cols != n || up.cols != 2 * n) fail("moe_glu_act: up must be [T, %lld] and out [T, %lld], of one dtype", (long long)(2 * n), (long long)n);
    if (logits.rows != up.rows || logits.cols != m.experts + (m.shared_gate ? 1 : 0)) fail("moe_glu_act: the logits must be [T, %d]", m.experts + (m.shared_gate ? 1 : 0));
    if (out.data == up.data) fail("moe_glu_act: out must not be up");
    check(mllm_moe_glu_act(up.data, i32(up.stride), static_cast<const float*>(logits.data), i32(logits.stride), m.experts, m.ff, m.shared_ff, m.top,
                           m.scale, m.sigmoid_router ? 1 : 0, m.limit, m.shared_limit, m.alpha, m.weight_on_input ? 1 : 0, m.shared_gate ? 1 : 0,
                           out.data, i32(out.stride), i32(up.rows), up.dtype, stream), "moe_glu_act");
}

void concat_cast(const Tensor2& a, const Tensor2& b, const Tensor2& out, hipStream_t stream) {
    need_f32(a, "concat_cast: a");
    need_f32(b, "concat_cast: b");
    need_act(out, "concat_cast: out");
    if (!a.contiguous() || !b.contiguous() || !out.contiguous() || a.rows != b.rows || a.cols != b.cols || out.rows != a.rows || out.cols != 2 * a.cols)
        fail("concat_cast: a and b must be contiguous [T, D] and out [T, 2 D]");
    check(mllm_concat_cast(static_cast<const float*>(a.data), static_cast<const float*>(b.data), i32(a.rows), i32(a.cols), out.data, out.dtype, stream),
          "concat_cast");
}

void glu_act(const Tensor2& gu, int act, const Tensor2& out, hipStream_t stream) {
    need_act(gu, "glu_act: the input");
    if (out.dtype != gu.dtype || out.rows != gu.rows || gu.cols != 2 * out.cols) fail("glu_act: out must be [T, F] for an input of [T, 2 F], of one dtype");
    check(mllm_glu_act(gu.data, i32(gu.stride), i32(gu.rows), i32(out.cols), act, out.data, i32(out.stride), gu.dtype, stream), "glu_act");
}

}  // namespace minillm
