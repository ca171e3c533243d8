// Checked dispatch of the RMS norms, the gated activation, the state-space mixer's kernels and latent
// attention (declared in ops.h beside the other ops).
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
}  // namespace

void rmsnorm(const Tensor2& x, const float* weight, float eps, int groups, const Tensor2* gate, const Tensor2& out,
             const int* rows, hipStream_t stream, int parts, size_t part_stride) {
    if (parts < 1 || (parts > 1 && part_stride < static_cast<size_t>(x.rows) * x.stride)) fail("rmsnorm: %d parts %zu floats apart do not hold the input", parts, part_stride);
    need_f32(x, "rmsnorm: the input");
    need_act(out, "rmsnorm out");
    if (weight == nullptr) fail("rmsnorm: the weight is missing");
    if (out.cols != x.cols) fail("rmsnorm: out has %lld columns, the input %lld", (long long)out.cols, (long long)x.cols);
    if (rows == nullptr && out.rows != x.rows) fail("rmsnorm: out has %lld rows, the input %lld", (long long)out.rows, (long long)x.rows);
    if (groups < 1 || x.cols % groups != 0) fail("rmsnorm: %lld columns do not split into %d equal parts", (long long)x.cols, groups);
    if (gate != nullptr) {
        need_f32(*gate, "rmsnorm: the gate");
        if (gate->rows != x.rows || gate->cols != x.cols) fail("rmsnorm: the gate must have the input's shape");
    }
    check(mllm_rmsnorm(static_cast<const float*>(x.data), i32(x.stride), rows, weight, gate ? static_cast<const float*>(gate->data) : nullptr,
                       gate ? i32(gate->stride) : 0, out.data, i32(out.stride), i32(out.rows), i32(x.cols), groups, eps, out.dtype, parts,
                       part_stride, stream),
          "rmsnorm");
}

void rms_linear(const Tensor2& x, const float* weight, float eps, const Tensor2& w, const float* bias, const Tensor2& out,
                int epilogue, const int* rows, void* tmp, hipStream_t stream) {
    need_f32(x, "rms_linear: the input");
    need_act(w, "rms_linear: w");
    const int64_t M = out.rows, K = x.cols;
    if (weight == nullptr) fail("rms_linear: the norm's weight is missing");
    if (w.cols != K || out.cols != w.rows) fail("rms_linear: rows of %lld do not fit a map of [%lld, %lld]", (long long)K, (long long)w.rows, (long long)w.cols);
    if (rows == nullptr && x.rows != M) fail("rms_linear: out has %lld rows, the input %lld", (long long)M, (long long)x.rows);
    const bool f32_out = epilogue == ADD_RESIDUAL || epilogue == STORE_F32;
    if (out.dtype != (f32_out ? F32 : w.dtype)) fail("rms_linear: out must be %s", dtype_name(f32_out ? F32 : w.dtype));
    // (more rows than that: the norm is a kernel of its own, as for the LayerNorm product)
    if (w.dtype == BF16 && M <= tuning().ln_fuse_max_rows && K % 8 == 0 && w.stride % 8 == 0 && x.contiguous() &&
        (reinterpret_cast<uintptr_t>(weight) & 15) == 0) {
        const int rc = mllm_rms_gemm_bf16(static_cast<const float*>(x.data), i32(x.stride), rows, weight, eps, w.data, i32(w.stride), bias,
                                          out.data, i32(out.stride), i32(M), i32(w.rows), i32(K), epilogue, stream);
        if (rc == 0) return;
        if (rc != -2) check(rc, "rms_linear");
    }
    if (tmp == nullptr) fail("rms_linear: these sizes need a buffer for the normalised rows");
    Tensor2 h(tmp, w.dtype, M, K);
    rmsnorm(x, weight, eps, 1, nullptr, h, rows, stream);
    linear(h, w, bias, out, epilogue, nullptr, stream);
}

void rmsnorm_add(const Tensor2& y, const float* weight, const float* scale, float mult, float eps, const Tensor2& x,
                 bool clear, hipStream_t stream) {
    need_f32(y, "rmsnorm_add: y");
    need_f32(x, "rmsnorm_add: x");
    if (weight == nullptr) fail("rmsnorm_add: the weight is missing");
    if (!y.contiguous() || !x.contiguous() || y.rows != x.rows || y.cols != x.cols)
        fail("rmsnorm_add: x and y must be contiguous float32 of one shape");
    check(mllm_rmsnorm_add(static_cast<float*>(y.data), weight, scale, mult, eps, static_cast<float*>(x.data), i32(x.rows), i32(x.cols),
                           clear ? 1 : 0, stream), "rmsnorm_add");
}

void glu_clamped(const Tensor2& gate, const Tensor2& up, float limit, float alpha, const Tensor2& out, hipStream_t stream) {
    need_act(gate, "glu_clamped gate");
    if (up.dtype != gate.dtype || out.dtype != gate.dtype || up.rows != gate.rows || up.cols != gate.cols || out.rows != gate.rows ||
        out.cols != gate.cols)
        fail("glu_clamped: gate, up and out must have one shape and dtype");
    check(mllm_glu_clamped(gate.data, i32(gate.stride), up.data, i32(up.stride), out.data, i32(out.stride), i32(gate.rows), i32(gate.cols),
                           limit, alpha, gate.dtype, stream), "glu_clamped");
}

void fill_zero(const Tensor2& x, hipStream_t stream) {
    need_f32(x, "fill_zero: the tensor");
    if (!x.contiguous()) fail("fill_zero: the tensor must be contiguous");
    // (whole 16-byte pieces: the arena hands out 256-byte steps, so the round-up stays inside the allocation)
    const size_t bytes = (static_cast<size_t>(x.rows) * x.cols * 4 + 15) / 16 * 16;
    check(mllm_fill_zero(x.data, bytes, stream), "fill_zero");
}

void conv_silu(const Tensor2& proj, int col0, const Tensor2& weight, const float* bias, const StateArgs& st,
               const Tensor2& out, hipStream_t stream) {
    need_f32(proj, "conv_silu: the input");
    need_f32(out, "conv_silu: out");
    need_f32(weight, "conv_silu: the taps");
    const int C = i32(weight.rows), taps = i32(weight.cols);
    if (!weight.contiguous() || bias == nullptr) fail("conv_silu: taps [channels, taps] contiguous and a bias are needed");
    if (taps < 1 || taps > 16) fail("conv_silu: %d taps are not supported (1 to 16)", taps);
    if (col0 < 0 || col0 + C > proj.cols || out.cols != C || out.rows != proj.rows)
        fail("conv_silu: %d channels from column %d do not fit rows of %lld, or out is not [%lld, %d]", C, col0, (long long)proj.cols,
             (long long)proj.rows, C);
    check_state(st, static_cast<size_t>(taps - 1) * C, "conv_silu");
    check(mllm_conv_silu(static_cast<const float*>(proj.data), i32(proj.stride), col0, C, static_cast<const float*>(weight.data), bias, taps,
                         st.token_seq, st.cu_q, st.state_slots, st.state, st.slot_floats, static_cast<float*>(out.data), i32(out.stride),
                         i32(proj.rows), st.n_seqs, st.write ? 1 : 0, stream), "conv_silu");
}

void ssm_scan(const Tensor2& xbc, const Tensor2& proj, int dt_col, const float* dt_bias, const float* A_log,
              const float* skip, const StateArgs& st, size_t scan_offset, int H, int P, int N, int G, const Tensor2& y,
              float* workspace, size_t workspace_floats, hipStream_t stream) {
    need_f32(xbc, "ssm_scan: x, B, C");
    need_f32(proj, "ssm_scan: the step sizes");
    need_f32(y, "ssm_scan: y");
    if (H < 1 || G < 1 || H % G != 0 || P < 1 || N < 1) fail("ssm_scan: %d heads, %d groups, %d x %d states are not supported", H, G, N, P);
    if (xbc.cols != static_cast<int64_t>(H) * P + 2 * G * N) fail("ssm_scan: x, B, C rows must be %d wide", H * P + 2 * G * N);
    if (dt_col < 0 || dt_col + H > proj.cols || proj.rows != xbc.rows) fail("ssm_scan: the step sizes lie outside their rows");
    if (y.rows != xbc.rows || y.cols != static_cast<int64_t>(H) * P) fail("ssm_scan: y must be [%lld, %d]", (long long)xbc.rows, H * P);
    if (dt_bias == nullptr || A_log == nullptr || skip == nullptr) fail("ssm_scan: dt_bias, A_log and D are needed");
    check_state(st, scan_offset + static_cast<size_t>(H) * P * N, "ssm_scan");
    const int T = i32(xbc.rows);
    // (a step whose longest portion is unknown is taken to have a long one)
    const int max_q = st.max_q_len > 0 ? st.max_q_len : T;
    if (workspace != nullptr && workspace_floats < ssm_scan_workspace_floats(T, st.n_seqs, H, P, N))
        fail("ssm_scan: the workspace holds %zu floats, %zu are needed", workspace_floats, ssm_scan_workspace_floats(T, st.n_seqs, H, P, N));
    check(mllm_ssm_scan(static_cast<const float*>(xbc.data), i32(xbc.stride), static_cast<const float*>(proj.data) + dt_col, i32(proj.stride),
                        dt_bias, A_log, skip, st.cu_q, st.state_slots, st.state, st.slot_floats, scan_offset, static_cast<float*>(y.data),
                        i32(y.stride), static_cast<size_t>(y.rows) * y.stride, T, st.n_seqs, max_q, H, P, N, G, st.write ? 1 : 0, workspace,
                        stream), "ssm_scan");
}

int ssm_scan_parts(int N) { return mllm_ssm_scan_parts(N); }

size_t ssm_scan_workspace_floats(int tokens, int n_seqs, int H, int P, int N) {
    return mllm_ssm_scan_workspace_floats(tokens, n_seqs, H, P, N);
}

static void check_shape(const LatentShape& sh, const char* what) {
    if (sh.n_heads < 1 || sh.plain_dim < 1 || sh.rot_dim < 0 || sh.value_dim < 1 || sh.kv_rank < 1 || sh.q_rank < 1)
        fail("%s: heads and sizes must be positive", what);
    if (sh.rot_dims < 0 || sh.rot_dims % 2 != 0 || sh.rot_dims > sh.rot_dim || sh.rot_dim % 2 != 0 || !(sh.rot_base > 0))
        fail("%s: %d of %d rotary columns (both even) and a positive base are needed", what, sh.rot_dims, sh.rot_dim);
}

static void check_pages(const LatentPages& pages, int dtype, const LatentShape& sh, const char* what) {
    const int E = sh.kv_rank + sh.rot_dim;
    if (pages.rows.dtype != dtype || !pages.rows.contiguous() || pages.rows.cols != E)
        fail("%s: the pages must be contiguous [rows, %d] %s", what, E, dtype_name(dtype));
    if (pages.page_size < 1 || pages.rows.rows % pages.page_size != 0) fail("%s: the page pool is not a whole number of pages", what);
    if (pages.latent_t.data != nullptr &&
        (pages.latent_t.dtype != dtype || !pages.latent_t.contiguous() || pages.latent_t.cols != sh.kv_rank || pages.latent_t.rows != pages.rows.rows))
        fail("%s: the transposed latent must be contiguous [rows, %d] %s", what, sh.kv_rank, dtype_name(dtype));
}

void latent_prepare(const Tensor2& dq, const float* wq, const Tensor2& cq, const Tensor2* dkv, const float* wkv,
                    const LatentPages* pages, const int* slots, const int* positions, const LatentShape& sh, hipStream_t stream) {
    check_shape(sh, "latent_prepare");
    need_f32(dq, "latent_prepare: the query latent");
    need_act(cq, "latent_prepare: cq");
    if (dq.cols != sh.q_rank || cq.cols != sh.q_rank || cq.rows != dq.rows || wq == nullptr)
        fail("latent_prepare: the query latent must be [T, %d] with its norm weight", sh.q_rank);
    if (dkv != nullptr) {
        need_f32(*dkv, "latent_prepare: the key/value latent");
        if (pages == nullptr || slots == nullptr || positions == nullptr || wkv == nullptr) fail("latent_prepare: pages, page rows, positions and the norm weight are needed");
        if (dkv->cols != sh.kv_rank + sh.rot_dim || dkv->rows != dq.rows) fail("latent_prepare: the key/value latent must be [T, %d]", sh.kv_rank + sh.rot_dim);
        check_pages(*pages, cq.dtype, sh, "latent_prepare");
    }
    check(mllm_latent_prepare(static_cast<const float*>(dq.data), i32(dq.stride), sh.q_rank, wq, cq.data, i32(cq.stride),
                              dkv ? static_cast<const float*>(dkv->data) : nullptr, dkv ? i32(dkv->stride) : 0, sh.kv_rank, sh.rot_dim, wkv,
                              dkv ? pages->rows.data : nullptr, dkv ? pages->latent_t.data : nullptr, dkv ? pages->page_size : 0, slots, positions,
                              i32(dq.rows), sh.eps, sh.rot_base, sh.rot_dims, cq.dtype, stream),
          "latent_prepare");
}

void latent_absorb(const Tensor2& q, const Tensor2& w_uk, const Tensor2& qa, const int* positions, const LatentShape& sh,
                   hipStream_t stream) {
    check_shape(sh, "latent_absorb");
    need_act(q, "latent_absorb: q");
    const int E = sh.kv_rank + sh.rot_dim;
    if (q.cols != static_cast<int64_t>(sh.n_heads) * (sh.plain_dim + sh.rot_dim)) fail("latent_absorb: q must be [T, %d]", sh.n_heads * (sh.plain_dim + sh.rot_dim));
    if (w_uk.dtype != q.dtype || w_uk.cols != static_cast<int64_t>(sh.n_heads) * sh.plain_dim || w_uk.rows != sh.kv_rank)
        fail("latent_absorb: the transposed key expansion must be [%d, %d] %s", sh.kv_rank, sh.n_heads * sh.plain_dim, dtype_name(q.dtype));
    if (qa.dtype != q.dtype || qa.rows != q.rows || qa.cols != static_cast<int64_t>(sh.n_heads) * E) fail("latent_absorb: qa must be [T, %d]", sh.n_heads * E);
    if (positions == nullptr) fail("latent_absorb: positions are needed");
    check(mllm_latent_absorb(q.data, i32(q.stride), w_uk.data, i32(w_uk.stride), qa.data, i32(qa.stride), positions, i32(q.rows), sh.n_heads,
                             sh.plain_dim, sh.rot_dim, sh.kv_rank, sh.rot_base, sh.rot_dims, q.dtype, stream), "latent_absorb");
}

// Rows x splits that a launch with split keys holds at most (its workspace is made for them).
constexpr long long LATENT_SPLIT_ROWS = 512 * 64;
size_t latent_attention_workspace_floats(int kv_rank) { return static_cast<size_t>(LATENT_SPLIT_ROWS) * (kv_rank + 2); }

void latent_attention(const Tensor2& qa, const LatentPages& pages, const LatentStep& step, float scale, int window,
                      const LatentShape& sh, const Tensor2& o_lat, float* workspace, size_t workspace_floats, hipStream_t stream) {
    check_shape(sh, "latent_attention");
    need_act(qa, "latent_attention: qa");
    const int E = sh.kv_rank + sh.rot_dim, T = i32(qa.rows);
    if (qa.cols != static_cast<int64_t>(sh.n_heads) * E) fail("latent_attention: qa must be [T, %d]", sh.n_heads * E);
    check_pages(pages, qa.dtype, sh, "latent_attention");
    if (o_lat.dtype != qa.dtype || o_lat.rows != qa.rows || o_lat.cols != static_cast<int64_t>(sh.n_heads) * sh.kv_rank)
        fail("latent_attention: the result must be [T, %d]", sh.n_heads * sh.kv_rank);
    if (step.block_tables == nullptr || step.token_seq == nullptr || step.positions == nullptr || step.max_blocks < 1)
        fail("latent_attention: block tables, token_seq and positions are needed");
    if (window < 0) fail("latent_attention: a negative window");
    // the matrix-core kernel: one workgroup per 64 (token, head) rows of a sequence
    if (tuning().latent_tiles && qa.dtype == BF16 && pages.latent_t.data != nullptr && step.cu_q != nullptr &&
        step.ctx_len != nullptr && step.n_seqs > 0 && qa.contiguous() && o_lat.contiguous()) {
        const bool single = step.max_q_len == 1 && T == step.n_seqs;        // one token a sequence: tiles are numbered directly
        const long long rows = static_cast<long long>(T) * sh.n_heads,
                        tiles = single ? static_cast<long long>(step.n_seqs) * ((sh.n_heads + 63) / 64) : rows / 64 + step.n_seqs;
        if (tiles < (1ll << 31)) {
            // Few workgroups (decoding): every row's key tiles are spread over several, so that about 256
            // workgroups stream the pages instead of one per sequence walking its tiles one after the other.
            const int keys = window > 0 ? std::min(window, std::max(step.max_ctx_len, 1)) : std::max(step.max_ctx_len, 1);
            int nsplit = 1;
            if (workspace != nullptr && tiles < 256) {
                nsplit = static_cast<int>(std::min<long long>({(keys + 63) / 64 + 1, 256 / tiles, 64, LATENT_SPLIT_ROWS / std::max<long long>(rows, 1)}));
                if (nsplit < 2 || static_cast<size_t>(rows) * nsplit * (sh.kv_rank + 2) > workspace_floats) nsplit = 1;
            }
            const int rc = mllm_latent_attention_tiles(qa.data, pages.rows.data, pages.latent_t.data, step.block_tables, step.max_blocks, step.cu_q,
                                                       step.ctx_len, step.n_seqs, static_cast<int>(tiles), sh.n_heads, sh.kv_rank, sh.rot_dim,
                                                       pages.page_size, scale, window, o_lat.data, static_cast<int>(rows), nsplit, workspace, single ? 1 : 0, stream);
            if (rc == 0) { tuning().seen.latent_tile_launches += 1; return; }
            if (rc != -2) check(rc, "latent_attention (tiles)");
        }
    }
    tuning().seen.latent_token_launches += 1;
    check(mllm_latent_attention(qa.data, i32(qa.stride), pages.rows.data, step.block_tables, step.max_blocks, step.token_seq, step.positions, T,
                                sh.n_heads, sh.kv_rank, sh.rot_dim, pages.page_size, scale, window, o_lat.data, i32(o_lat.stride), qa.dtype, stream),
          "latent_attention");
}

void latent_expand(const Tensor2& o_lat, const Tensor2& w_uv, const Tensor2& out, const LatentShape& sh, hipStream_t stream) {
    check_shape(sh, "latent_expand");
    need_act(o_lat, "latent_expand: the attention result");
    if (o_lat.cols != static_cast<int64_t>(sh.n_heads) * sh.kv_rank) fail("latent_expand: the attention result must be [T, %d]", sh.n_heads * sh.kv_rank);
    if (w_uv.dtype != o_lat.dtype || w_uv.rows != static_cast<int64_t>(sh.n_heads) * sh.value_dim || w_uv.cols != sh.kv_rank)
        fail("latent_expand: the value expansion must be [%d, %d] %s", sh.n_heads * sh.value_dim, sh.kv_rank, dtype_name(o_lat.dtype));
    if (out.dtype != o_lat.dtype || out.rows != o_lat.rows || out.cols != w_uv.rows) fail("latent_expand: out must be [T, %lld]", (long long)w_uv.rows);
    check(mllm_latent_expand(o_lat.data, i32(o_lat.stride), w_uv.data, i32(w_uv.stride), out.data, i32(out.stride), i32(o_lat.rows), sh.n_heads,
                             sh.value_dim, sh.kv_rank, o_lat.dtype, stream), "latent_expand");
}

}  // namespace minillm
