// Softmax attention whose scores are shaped before the softmax, as one mixer with its choices as parameters.
#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int64_t n) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("scored_attention: '%s' must be contiguous float32 [%lld]", key, (long long)n);
    return static_cast<const float*>(t.data);
}

// With h the mixer's input and one joined input projection whose rows are [queries: heads * dim | keys: kv_heads * dim |
// values: kv_heads * value_dim (absent with values_from_keys) | gate: heads * value_dim (only with gated)]:
//   q, k   with qk_conv ([(heads + kv_heads) * dim, taps]) first a short causal convolution over time on every channel
//          of the projected queries and keys (the last tap the token's own; the last taps - 1 projected rows of a request
//          are carried in its state slot), then
//          RMS-normed (qk_norm "head": per head, one weight [dim] shared by the heads; "row": over all heads at once,
//          weights as wide as the projections; "none"), then the first rot_dims columns of every head turned by the
//          token's position (column i pairs with i + rot_dims / 2, or with rot_interleaved column 2i with 2i + 1; angle
//          p * rot_base^(-2i / rot_dims)); qk_norm "unit_after": every head scaled to unit root mean square BEHIND the
//          turn, without a weight
//   v      its own projection, or (values_from_keys) the keys as projected (behind the convolution), before norm and turn
//   score  scale (q . k);  softcap > 0: softcap tanh(score / softcap);  with r1, r2 (one number per head each):
//          minus r1 ln(1 + r2 (i - j));  or with distance_slope (one number per head): minus slope (i - j)
//   mask   causal, within a sliding window (0 <= i - j < window; with keep_first also the sequence's first keep_first
//          positions, at their true distances) or within the chunk of `chunk` positions that holds i
//   weight softmax(score) over the visible keys, with `sink` (one number per head) one more term exp(sink) in the
//          denominator that has no value; or, with sigmoid_weights, sigmoid(score + score_bias[head]) for every
//          visible key on its own, not normalised over the keys
//   out    W_o (concat_heads(sum_j weight_j v_j) * sigmoid(gate)) (+ bias), added into the stream; with gate_per_head
//          the gate projection has one row per head instead of one per value column.
// Query head h reads key/value head h / (heads / kv_heads). Normed and turned keys and the values live in pages.
// With shared_kv the mixer has no keys and values of its own: the joined projection holds queries (and gate) only, and
// the call of the execution order reads the pages that another layer's mixer of the same head counts wrote.
// Parameters: heads, kv_heads, dim, value_dim, scale, softcap, window, keep_first, chunk, rot_dims, rot_base,
// rot_interleaved, eps, dtype, values_from_keys, gated, gate_per_head, sigmoid_weights, shared_kv; string qk_norm;
// tensors in.weight, out.weight, [in.bias, out.bias], [q.norm, k.norm], [r1, r2], [distance_slope], [sink],
// [score_bias], [qk_conv].
class ScoredAttention final : public Mixer {
public:
    explicit ScoredAttention(const Params& p) {
        sh_.n_heads = p.integer("heads");
        sh_.n_kv_heads = p.integer("kv_heads");
        sh_.dim = p.integer("dim");
        sh_.value_dim = p.integer("value_dim");
        sh_.scale = static_cast<float>(p.number("scale"));
        sh_.softcap = static_cast<float>(p.number("softcap", 0.0));
        sh_.window = static_cast<int>(p.number("window", 0));
        sh_.chunk = static_cast<int>(p.number("chunk", 0));
        sh_.rot_dims = static_cast<int>(p.number("rot_dims", 0));
        sh_.rot_base = p.number("rot_base", 10000.0);
        sh_.rot_interleaved = p.number("rot_interleaved", 0) != 0;
        sh_.keep_first = static_cast<int>(p.number("keep_first", 0));
        shared_kv_ = p.number("shared_kv", 0) != 0;
        sh_.eps = static_cast<float>(p.number("eps", 1e-6));
        dtype_ = p.integer("dtype");
        values_from_keys_ = p.number("values_from_keys", 0) != 0;
        gated_ = p.number("gated", 0) != 0;
        sh_.gate_per_head = gated_ && p.number("gate_per_head", 0) != 0;
        sh_.sigmoid_weights = p.number("sigmoid_weights", 0) != 0;
        const int H = sh_.n_heads, G = sh_.n_kv_heads, d = sh_.dim, dv = sh_.value_dim;
        if (H < 1 || G < 1 || H % G != 0 || d < 1 || dv < 1) fail("scored_attention: %d heads over %d key/value heads of %d / %d do not fit", H, G, d, dv);
        if (sh_.window < 0 || sh_.chunk < 0 || (sh_.window > 0 && sh_.chunk > 0)) fail("scored_attention: a window or a chunk, not both");
        if (sh_.keep_first < 0 || (sh_.keep_first > 0 && sh_.window <= 0)) fail("scored_attention: kept first positions go with a sliding window");
        if (values_from_keys_ && dv != d) fail("scored_attention: values taken from the keys have the keys' width, %d, not %d", d, dv);
        if (sh_.rot_dims < 0 || sh_.rot_dims % 2 != 0 || sh_.rot_dims > d) fail("scored_attention: %d turned columns of %d: even and at most the head", sh_.rot_dims, d);
        const std::string& mode = p.string("qk_norm");
        if (mode == "none") sh_.norm_mode = 0;
        else if (mode == "head") sh_.norm_mode = 1;
        else if (mode == "row") sh_.norm_mode = 2;
        else if (mode == "unit_after") sh_.norm_mode = 3;
        else fail("scored_attention: qk_norm '%s' is not one of none, head, row, unit_after", mode.c_str());
        if (shared_kv_ && (sh_.norm_mode == 2 || values_from_keys_)) fail("scored_attention: a mixer without keys of its own has no row norm over them and takes no values from them");
        if (sh_.norm_mode == 1) { sh_.q_norm = f32_vector(p, "q.norm", d); sh_.k_norm = f32_vector(p, "k.norm", d); }
        if (sh_.norm_mode == 2) { sh_.q_norm = f32_vector(p, "q.norm", static_cast<int64_t>(H) * d); sh_.k_norm = f32_vector(p, "k.norm", static_cast<int64_t>(G) * d); }
        if (p.weights_or_null("r1") != nullptr) { sh_.r1 = f32_vector(p, "r1", H); sh_.r2 = f32_vector(p, "r2", H); }
        if (p.weights_or_null("distance_slope") != nullptr) {
            if (sh_.r1 != nullptr) fail("scored_attention: a linear or a logarithmic distance bias, not both");
            sh_.slope = f32_vector(p, "distance_slope", H);
        }
        if (p.weights_or_null("sink") != nullptr) {
            if (sh_.sigmoid_weights) fail("scored_attention: a sink stands in a softmax's denominator; sigmoid weights have none");
            sh_.sink = f32_vector(p, "sink", H);
        }
        if (p.weights_or_null("score_bias") != nullptr) {
            if (!sh_.sigmoid_weights) fail("scored_attention: a score bias per head goes with sigmoid weights only (a softmax cancels it)");
            sh_.score_bias = f32_vector(p, "score_bias", H);
        }
        in_ = Linear(p.weights("in.weight"), p.weights_or_null("in.bias"));
        out_ = Linear(p.weights("out.weight"), p.weights_or_null("out.bias"));
        k_col_ = shared_kv_ ? -1 : H * d;
        v_col_ = (values_from_keys_ || shared_kv_) ? -1 : k_col_ + G * d;
        gate_col_ = shared_kv_ ? H * d : k_col_ + G * d + (values_from_keys_ ? 0 : G * dv);
        if (const Tensor2* c = p.weights_or_null("qk_conv")) {
            if (shared_kv_) fail("scored_attention: the convolution runs over queries and keys; a mixer without keys of its own has none");
            if (c->dtype != F32 || !c->contiguous() || c->rows != static_cast<int64_t>(H + G) * d || c->cols < 1 || c->cols > 16)
                fail("scored_attention: 'qk_conv' must be contiguous float32 [%d, 1 to 16 taps]", (H + G) * d);
            conv_ = *c;
            conv_bytes_ = static_cast<size_t>(c->cols - 1) * c->rows * 4;
        }
        if (in_.out_features() != gate_col_ + (gated_ ? (sh_.gate_per_head ? H : H * dv) : 0) || out_.in_features() != H * dv)
            fail("scored_attention: the projections' shapes do not fit %d heads of %d / %d over %d key/value heads", H, d, dv, G);
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        run(h, step, cache, x, write, arena, s, ADD_RESIDUAL);
    }
    void forward_set(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                     hipStream_t s) const override {
        run(h, step, cache, x, write, arena, s, STORE_F32);
    }
    void run(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
             hipStream_t s, int out_epilogue) const {
        if (!cache.has_pages()) fail("scored_attention needs a cache of pages");
        if (write == shared_kv_) fail(shared_kv_ ? "scored_attention without keys of its own reads another call's cache: it cannot write one"
                                                 : "scored_attention writes its own keys and values: it cannot read another call's cache");
        const int T = step.n_tokens, g = cache.group, N = in_.out_features(), ld = (N + 3) / 4 * 4;
        Tensor2 proj(arena.take(static_cast<size_t>(T) * ld * 4), F32, T, N, ld);
        h.linear(in_, proj, STORE_F32, nullptr, arena, s);
        Tensor2 q = arena.tensor(dtype_, T, sh_.n_heads * sh_.dim);
        if (conv_.data != nullptr) {
            // the convolution over the projected queries and keys (they lie side by side in front of the rows)
            if (conv_bytes_ > 0 && (!cache.has_state() || cache.state_bytes < conv_bytes_)) fail("scored_attention with a convolution needs %zu bytes of state per request", conv_bytes_);
            const int C = static_cast<int>(conv_.rows);
            Tensor2 qk(arena.take(static_cast<size_t>(T) * C * 4), F32, T, C);
            StateArgs st;
            st.token_seq = step.token_seq; st.cu_q = step.cu_q; st.state_slots = step.state_slots; st.n_seqs = step.n_seqs;
            st.max_q_len = step.max_q_len; st.state = static_cast<float*>(cache.state); st.slot_floats = cache.slot_bytes / 4;
            st.n_slots = cache.n_slots; st.write = write;
            conv_residual(Tensor2(proj.data, F32, T, C, ld), conv_, st, qk, s, false);      // (four channels a thread where the sizes allow)
            qk_prepare(qk, 0, k_col_, v_col_, sh_, step.positions, step.slots[g], q, cache.k_pages, cache.v_pages, s);
        } else {
            qk_prepare(proj, 0, k_col_, v_col_, sh_, step.positions, step.slots[g], q, cache.k_pages, cache.v_pages, s);
        }
        StageTimes::get().mark("qkv", s);
        ScoredStep st;
        st.block_tables = step.block_tables[g]; st.max_blocks = step.max_blocks[g]; st.n_seqs = step.n_seqs; st.max_q_len = step.max_q_len;
        st.max_ctx_len = step.max_ctx_len; st.page_size = cache.page_size; st.token_seq = step.token_seq; st.positions = step.positions;
        st.cu_q = step.cu_q; st.ctx_len = step.ctx_len; st.n_single = step.n_single;
        Tensor2 o = arena.tensor(dtype_, T, sh_.n_heads * sh_.value_dim);
        scored_attention(q, cache.k_pages, cache.v_pages, st, sh_, gated_ ? &proj : nullptr, gate_col_, o, s);
        StageTimes::get().mark("attention", s);
        out_(o, x, out_epilogue, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * ((in_.out_features() + 4) * 4 + conv_.rows * 4 + (sh_.n_heads * (sh_.dim + sh_.value_dim) + in_.in_features()) * dtype_size(dtype_)) + 4096;
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        // (a chunked mask keeps its pages: only a sliding window tells the manager what it may take back)
        n.kind = 1; n.n_kv_heads = sh_.n_kv_heads; n.head_dim = sh_.dim; n.value_dim = sh_.value_dim; n.window = sh_.window;
        n.keep_first = sh_.keep_first;
        if (conv_bytes_ > 0) { n.kind |= 2; n.state_bytes = conv_bytes_; }
        return n;
    }
    void reserve(int max_seqs, hipStream_t s) const override {
        reserve_attention_scratch((max_seqs + 7) / 8 * 8, sh_.n_heads, sh_.dim, s);
        reserve_linear_scratch(s);
    }
    void add_cost(StepCost& c) const override {
        in_.add_cost(c);
        out_.add_cost(c);
        c.attention_flops_per_key += 2.0 * sh_.n_heads * (sh_.dim + sh_.value_dim);
        if (conv_.data != nullptr) { c.weight_bytes += 4.0 * conv_.rows * conv_.cols; c.flops_per_token += 2.0 * conv_.rows * conv_.cols; }
    }

private:
    ScoredShape sh_;
    int dtype_ = BF16, k_col_ = 0, v_col_ = 0, gate_col_ = 0;
    bool values_from_keys_ = false, gated_ = false, shared_kv_ = false;
    Linear in_, out_;
    Tensor2 conv_;                   // [(heads + kv_heads) * dim, taps], or empty: no convolution
    size_t conv_bytes_ = 0;
};

}  // namespace

void register_scored_attention() {
    register_mixer("scored_attention", [](const Params& p) { return std::unique_ptr<Mixer>(new ScoredAttention(p)); });
}

}  // namespace minillm
