// The gated linear recurrence (HGRN2) as a mixer, mixers that run side by side, the gated feed-forward with
// biases, the token table with a norm behind it, and the stream step that mixes the embedding's output back in.
#include <algorithm>

#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int64_t n, const char* who) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("%s: '%s' must be contiguous float32 [%lld]", who, key, (long long)n);
    return static_cast<const float*>(t.data);
}

// HGRN2: linear attention in which the forget gate also decides what is written. One joined input projection
// whose rows are [q: heads * dim | f: heads * dim | v: heads * value_dim]; per head, token by token,
//   f = lower + (1 - lower) sigmoid(f_raw + f_bias);  S <- diag(f) S + (1 - f) v^T;  o = S^T silu(q_raw)
// then every head's o is RMS-normed over value_dim (weight per column of the concatenated heads: a weight that the
// heads share is handed over repeated), and W_o of the concatenated heads is added into the stream. The state
// ([heads][dim][value_dim], fp32) is carried per request in a state slot; gates, state and norm are fp32 in both
// precisions, the two projections run in the compute dtype.
// Parameters: heads, dim, value_dim, eps, dtype; tensors in.weight, f.bias (optional), lower, norm.weight, out.weight.
class Hgrn2Mixer final : public Mixer {
public:
    explicit Hgrn2Mixer(const Params& p) {
        H_ = p.integer("heads"); d_ = p.integer("dim"); dv_ = p.integer("value_dim");
        eps_ = static_cast<float>(p.number("eps"));
        dtype_ = p.integer("dtype");
        if (H_ < 1 || d_ < 1 || dv_ < 1) fail("hgrn2: heads and sizes must be positive");
        in_ = Linear(p.weights("in.weight"), nullptr);
        out_ = Linear(p.weights("out.weight"), nullptr);
        if (in_.out_features() != 2 * H_ * d_ + H_ * dv_ || out_.in_features() != H_ * dv_)
            fail("hgrn2: the projections' shapes do not fit %d heads of %d / %d", H_, d_, dv_);
        if (p.weights_or_null("f.bias") != nullptr) f_bias_ = f32_vector(p, "f.bias", static_cast<int64_t>(H_) * d_, "hgrn2");
        lower_ = f32_vector(p, "lower", static_cast<int64_t>(H_) * d_, "hgrn2");
        norm_ = f32_vector(p, "norm.weight", static_cast<int64_t>(H_) * dv_, "hgrn2");
        state_floats_ = static_cast<size_t>(H_) * d_ * dv_;
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
        if (!cache.has_state() || cache.state_bytes < state_floats_ * 4) fail("hgrn2 needs a state of %zu floats per request", state_floats_);
        const int T = step.n_tokens, N = in_.out_features(), ld = (N + 3) / 4 * 4, inner = H_ * dv_;
        Tensor2 proj(arena.take(static_cast<size_t>(T) * ld * 4), F32, T, N, ld);
        h.linear(in_, proj, STORE_F32, nullptr, arena, s);
        StageTimes::get().mark("in_proj", s);
        StateArgs st;
        st.token_seq = step.token_seq; st.cu_q = step.cu_q; st.state_slots = step.state_slots; st.n_seqs = step.n_seqs;
        st.max_q_len = step.max_q_len; st.state = static_cast<float*>(cache.state); st.slot_floats = cache.slot_bytes / 4;
        st.n_slots = cache.n_slots; st.write = write;
        // (the scan leaves its result as shares, one per slice of the key channels; the norm adds them)
        const int parts = hgrn2_parts(d_);
        Tensor2 y(arena.take(static_cast<size_t>(parts) * T * inner * 4), F32, T, inner);
        // (portions longer than a chunk are scanned chunk by chunk side by side: room for the chunks' states)
        const size_t ws_floats = step.max_q_len > hgrn2_chunk() ? hgrn2_workspace_floats(T, step.n_seqs, H_, d_, dv_) : 0;
        float* ws = ws_floats ? static_cast<float*>(arena.take(ws_floats * 4)) : nullptr;
        hgrn2_scan(proj, 0, H_ * d_, 2 * H_ * d_, f_bias_, lower_, st, 0, H_, d_, dv_, y, ws, ws_floats, s);
        StageTimes::get().mark("scan", s);
        Tensor2 normed = arena.tensor(dtype_, T, inner);
        rmsnorm(y, norm_, eps_, H_, nullptr, normed, nullptr, s, parts, static_cast<size_t>(T) * inner);
        out_(normed, x, out_epilogue, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * ((in_.out_features() + 4) * 4 + hgrn2_parts(d_) * H_ * dv_ * 4 + (H_ * dv_ + in_.in_features()) * dtype_size(dtype_)) +
               // (every sequence of a step adds at most one chunk that is not full; a step holds at most as many
               // sequences as tokens)
               hgrn2_workspace_floats(tokens, std::min(tokens, 256), H_, d_, dv_) * 4 + 8192;
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = 2;
        n.state_bytes = state_floats_ * 4;
        return n;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override {
        in_.add_cost(c);
        out_.add_cost(c);
        c.weight_bytes += 4.0 * (3.0 * H_ * d_ + H_ * dv_);
        c.flops_per_token += 5.0 * H_ * d_ * dv_;          // the state's update and readout
    }

private:
    int H_ = 0, d_ = 0, dv_ = 0, dtype_ = BF16;
    float eps_ = 1e-6f;
    Linear in_, out_;
    const float *f_bias_ = nullptr, *lower_ = nullptr, *norm_ = nullptr;
    size_t state_floats_ = 0;
};

// Mixers side by side on the same input: x += (1 / n) sum_k rmsnorm(mixer_k(h)) * weight_k, every mixer's output
// RMS-normed over the stream's width with a weight of its own before the mean is taken. Each mixer sets an fp32
// buffer of the stream's shape (Mixer::forward_set). At most one of them may keep pages; their states lie one behind the
// other in the layer's state slot. Parameters: size, eps; mixers; tensors norm0, norm1, ... and optionally
// norms (the same weights one behind the other: the norms and the mean then run in one kernel).
class ParallelMixers final : public Mixer {
public:
    explicit ParallelMixers(const Params& p) : mixers_(p.mixers) {
        size_ = p.integer("size");
        eps_ = static_cast<float>(p.number("eps"));
        if (mixers_.size() < 2) fail("parallel mixers: at least two mixers are needed");
        int with_pages = 0;
        for (size_t k = 0; k < mixers_.size(); ++k) {
            if (!mixers_[k]) fail("parallel mixers: mixer %zu is missing", k);
            norms_.push_back(f32_vector(p, ("norm" + std::to_string(k)).c_str(), size_, "parallel mixers"));
            if (mixers_[k]->cache_need().kind & 1) with_pages += 1;
        }
        if (with_pages > 1) fail("parallel mixers: only one of the mixers may keep pages");
        // (the weights one behind the other in one tensor: all norms and the mean in one kernel)
        if (const Tensor2* j = p.weights_or_null("norms")) {
            if (j->dtype != F32 || !j->contiguous() || j->rows * j->cols != static_cast<int64_t>(size_) * static_cast<int64_t>(mixers_.size()))
                fail("parallel mixers: 'norms' must be contiguous float32 [%zu * %d]", mixers_.size(), size_);
            joined_norms_ = static_cast<const float*>(j->data);
        }
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        const int n = static_cast<int>(mixers_.size());
        if (x.cols != size_) fail("parallel mixers of width %d were handed a stream of %lld", size_, (long long)x.cols);
        Tensor2 all = arena.tensor(F32, x.rows * n, x.cols);          // (every mixer sets its own share)
        size_t state_at = 0;
        for (int k = 0; k < n; ++k) {
            const CacheNeed need = mixers_[k]->cache_need();
            CacheView mine = cache;
            mine.kind = 0;
            if (need.kind & 1) {
                if (!cache.has_pages()) fail("parallel mixers: mixer %d needs pages", k);
                mine.kind |= 1;
            }
            if (need.kind & 2) {
                if (!cache.has_state() || cache.state_bytes < state_at + need.state_bytes) fail("parallel mixers: mixer %d needs %zu bytes of state", k, need.state_bytes);
                mine.kind |= 2;
                mine.state = static_cast<char*>(cache.state) + state_at;
                mine.state_bytes = need.state_bytes;
                state_at += (need.state_bytes + 15) / 16 * 16;
            }
            const size_t mark = arena.mark();
            mixers_[k]->forward_set(h, step, mine, all.row_range(x.rows * k, x.rows), write, arena, s);
            arena.release(mark);
        }
        if (joined_norms_ != nullptr && n <= 4 && x.cols <= 2048) rmsnorm_add_many(all, joined_norms_, n, 1.0f / n, eps_, x, s);
        else for (int k = 0; k < n; ++k) rmsnorm_add(all.row_range(x.rows * k, x.rows), norms_[k], nullptr, 1.0f / n, eps_, x, false, s);
        StageTimes::get().mark("mix", s);
    }
    size_t workspace_bytes(int tokens) const override {
        size_t most = 0;
        for (const auto& m : mixers_) most = std::max(most, m->workspace_bytes(tokens));
        return most + static_cast<size_t>(tokens) * size_ * 4 * mixers_.size() + 1024;
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        for (const auto& m : mixers_) {
            const CacheNeed one = m->cache_need();
            if (one.kind & 1) { n.n_kv_heads = one.n_kv_heads; n.head_dim = one.head_dim; n.value_dim = one.value_dim; n.window = one.window; }
            if (one.kind & 2) n.state_bytes += (one.state_bytes + 15) / 16 * 16;
            n.kind |= one.kind;
        }
        return n;
    }
    void reserve(int max_seqs, hipStream_t s) const override { for (const auto& m : mixers_) m->reserve(max_seqs, s); }
    void add_cost(StepCost& c) const override {
        for (const auto& m : mixers_) m->add_cost(c);
        c.weight_bytes += 4.0 * size_ * mixers_.size();
    }

private:
    std::vector<std::shared_ptr<const Mixer>> mixers_;
    std::vector<const float*> norms_;
    const float* joined_norms_ = nullptr;
    int size_ = 0;
    float eps_ = 1e-6f;
};

// x += W_down(act(W_gate h + b_gate) * (W_up h + b_up)) + b_down. Gate and up are one joined product, rows
// [gate: ff | up: ff]. Parameters: dtype, string activation (gelu_tanh, silu); tensors gate_up.weight, gate_up.bias
// (optional), down.weight, down.bias (optional).
class GatedMLP final : public FeedForward {
public:
    explicit GatedMLP(const Params& p) {
        dtype_ = p.integer("dtype");
        const std::string& act = p.string("activation");
        if (act == "gelu_tanh") act_ = GELU_TANH;
        else if (act == "silu") act_ = GLU_SILU;
        else fail("gated_mlp: unknown activation '%s' (known: gelu_tanh, silu)", act.c_str());
        gate_up_ = Linear(p.weights("gate_up.weight"), p.weights_or_null("gate_up.bias"));
        down_ = Linear(p.weights("down.weight"), p.weights_or_null("down.bias"));
        if (gate_up_.out_features() != 2 * down_.in_features()) fail("gated_mlp: the products' shapes do not fit");
    }
    void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        Pending p;
        begin(h, step, arena, s, p);
        finish(p, step, x, arena, s);
    }
    bool begin(NormedInput& h, const StepView& step, Arena& arena, hipStream_t s, Pending& pending) const override {
        pending.a = arena.tensor(dtype_, step.n_tokens, 2 * down_.in_features());
        h.linear(gate_up_, pending.a, STORE, nullptr, arena, s);
        StageTimes::get().mark("fc1", s);
        return true;
    }
    void finish(const Pending& pending, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        Tensor2 a = arena.tensor(dtype_, step.n_tokens, down_.in_features());
        glu_act(pending.a, act_, a, s);
        down_(a, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("fc2", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * (3 * down_.in_features() + gate_up_.in_features()) * dtype_size(dtype_) + 2048;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override { gate_up_.add_cost(c); down_.add_cost(c); }

private:
    int dtype_ = BF16, act_ = GELU_TANH;
    Linear gate_up_, down_;
};

// x[t,:] = rmsnorm(table[id[t],:]) * weight: a token table with an RMS norm behind it.
// Parameters: eps; tensors table, norm.weight.
class NormedTokenTable final : public Embedding {
public:
    explicit NormedTokenTable(const Params& p) : table_(p.weights("table")) {
        eps_ = static_cast<float>(p.number("eps"));
        weight_ = f32_vector(p, "norm.weight", table_.cols, "normed_token_table");
    }
    int vocab_size() const override { return static_cast<int>(table_.rows); }
    int hidden_size() const override { return static_cast<int>(table_.cols); }
    void forward(const StepView& step, const PositionEncoding* position, const Tensor2& x, hipStream_t s) const override {
        embed(step.token_ids, step.positions, table_, position ? position->table() : nullptr, x, s, &step.fed);
        rmsnorm(x, weight_, eps_, 1, nullptr, x, nullptr, s);          // in place: a lane writes what it alone has read
    }
    bool resolves_fed_tokens() const override { return true; }
    void add_cost(StepCost& c) const override { c.weight_bytes += 4.0 * table_.cols; }

private:
    Tensor2 table_;         // [V, D]
    const float* weight_ = nullptr;
    float eps_ = 1e-6f;
};

// x <- W [x; x0] + step[pass]: the stream and the embedding's output side by side through one linear map
// (weight [width, 2 width], the stream's columns first), plus one vector per pass. Parameters: dtype; tensors
// weight, steps ([passes, width] fp32).
class EmbeddingMix final : public StreamStep {
public:
    explicit EmbeddingMix(const Params& p) {
        dtype_ = p.integer("dtype");
        map_ = Linear(p.weights("weight"), nullptr);
        if (map_.in_features() != 2 * map_.out_features()) fail("embedding_mix: the map must be [width, 2 width]");
        steps_ = p.weights("steps");
        if (steps_.dtype != F32 || !steps_.contiguous() || steps_.cols != map_.out_features() || steps_.rows < 1)
            fail("embedding_mix: the steps must be contiguous float32 [passes, %d]", map_.out_features());
    }
    void forward(const Tensor2& x, const Tensor2& x0, int pass, const StepView&, Arena& arena, hipStream_t s) const override {
        if (x0.data == nullptr || x.cols != map_.out_features()) fail("embedding_mix needs the embedding's output beside a stream of width %d", map_.out_features());
        if (pass < 0 || pass >= steps_.rows) fail("embedding_mix: pass %d of %lld", pass, (long long)steps_.rows);
        Tensor2 both = arena.tensor(dtype_, x.rows, 2 * x.cols);
        concat_cast(x, x0, both, s);
        linear(both, map_.weight, static_cast<const float*>(steps_.data) + static_cast<size_t>(pass) * steps_.cols, x, STORE_F32, nullptr, s);
    }
    size_t workspace_bytes(int tokens) const override { return static_cast<size_t>(tokens) * map_.in_features() * dtype_size(dtype_) + 512; }
    bool wants_embedding_output() const override { return true; }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override { map_.add_cost(c); c.weight_bytes += 4.0 * steps_.cols; }

private:
    int dtype_ = BF16;
    Linear map_;
    Tensor2 steps_;
};

}  // namespace

void register_recurrent_parts() {
    register_mixer("hgrn2", [](const Params& p) { return std::unique_ptr<Mixer>(new Hgrn2Mixer(p)); });
    register_mixer("parallel", [](const Params& p) { return std::unique_ptr<Mixer>(new ParallelMixers(p)); });
    register_feed_forward("gated_mlp", [](const Params& p) { return std::unique_ptr<FeedForward>(new GatedMLP(p)); });
    register_embedding("normed_token_table", [](const Params& p) { return std::unique_ptr<Embedding>(new NormedTokenTable(p)); });
    register_stream_step("embedding_mix", [](const Params& p) { return std::unique_ptr<StreamStep>(new EmbeddingMix(p)); });
}

}  // namespace minillm
