// Linear attention with a decay per key channel as a mixer, the feed-forward of routed experts, and the stream step
// that hands on a weighted sum of all streams so far.
#include <algorithm>
#include <cmath>

#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int64_t n, const char* who) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("%s: '%s' must be contiguous float32 [%lld]", who, key, (long long)n);
    return static_cast<const float*>(t.data);
}

// Linear attention without a softmax or a denominator: per head, token by token,
//   S <- diag(f) S + k v^T,   o = S^T q
// with q = q_scale * turn(W_q h), k = k_scale * turn(W_k h), v = W_v h. The turn is rotary over the first rot_dims
// columns of every head (column i pairs with i + rot_dims / 2, angle p * rot_base^(-2i / rot_dims)); rot_dims 0: none.
// The decays f are either one constant per head (tensor head_decay [heads]) or, per token and key channel,
//   f = sigmoid(W_2 (W_1 h) + b_2)^(1 / tau)
// with a low-rank map (decay.weight [heads * dim, rank], decay.bias, the rank values of W_1 h come out of the joined
// input projection). Every head's o is RMS-normed over value_dim (norm.weight per column of the concatenated heads, or
// none), multiplied by silu(W_g h), and W_o of the concatenated heads goes into the stream. One joined input
// projection whose rows are [q: heads * dim | k: heads * dim | v: heads * value_dim | g: heads * value_dim | W_1: rank].
// The state ([heads][dim][value_dim], fp32) is carried per request in a state slot; the projection's result, turn,
// decays, state, sums, norm and gate are fp32 in both precisions, the two projections run in the compute dtype.
// Parameters: heads, dim, value_dim, eps, dtype, q_scale, k_scale, rot_dims, rot_base, tau; tensors in.weight,
// out.weight, [norm.weight], head_decay | decay.weight (+ decay.bias).
class LinearAttention final : public Mixer {
public:
    explicit LinearAttention(const Params& p) {
        H_ = p.integer("heads"); d_ = p.integer("dim"); dv_ = p.integer("value_dim");
        eps_ = static_cast<float>(p.number("eps"));
        dtype_ = p.integer("dtype");
        q_scale_ = static_cast<float>(p.number("q_scale", 1.0));
        k_scale_ = static_cast<float>(p.number("k_scale", 1.0));
        rot_dims_ = static_cast<int>(p.number("rot_dims", 0));
        rot_base_ = p.number("rot_base", 10000.0);
        if (H_ < 1 || d_ < 1 || dv_ < 1) fail("linear_attention: heads and sizes must be positive");
        if (rot_dims_ < 0 || rot_dims_ % 2 != 0 || rot_dims_ > d_) fail("linear_attention: %d turned columns of %d: even and at most the head", rot_dims_, d_);
        in_ = Linear(p.weights("in.weight"), nullptr);
        out_ = Linear(p.weights("out.weight"), nullptr);
        if (const Tensor2* w = p.weights_or_null("decay.weight")) {
            if (w->dtype != F32 || !w->contiguous() || w->rows != static_cast<int64_t>(H_) * d_ || w->cols < 1)
                fail("linear_attention: 'decay.weight' must be contiguous float32 [%d, rank]", H_ * d_);
            decay_map_ = *w;
            rank_ = static_cast<int>(w->cols);
            if (p.weights_or_null("decay.bias") != nullptr) decay_bias_ = f32_vector(p, "decay.bias", static_cast<int64_t>(H_) * d_, "linear_attention");
            tau_ = static_cast<float>(p.number("tau"));
            if (!(tau_ > 0.f)) fail("linear_attention: tau must be positive");
        } else {
            head_decay_ = f32_vector(p, "head_decay", H_, "linear_attention");
        }
        if (p.weights_or_null("norm.weight") != nullptr) norm_ = f32_vector(p, "norm.weight", static_cast<int64_t>(H_) * dv_, "linear_attention");
        k_col_ = H_ * d_; v_col_ = 2 * H_ * d_; g_col_ = v_col_ + H_ * dv_; a_col_ = g_col_ + H_ * dv_;
        if (in_.out_features() != a_col_ + rank_ || out_.in_features() != H_ * dv_)
            fail("linear_attention: the projections' shapes do not fit %d heads of %d / %d (rank %d)", H_, d_, dv_, rank_);
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
        if (!cache.has_state() || cache.state_bytes < state_floats_ * 4) fail("linear_attention needs a state of %zu floats per request", state_floats_);
        const int T = step.n_tokens, N = in_.out_features(), ld = (N + 3) / 4 * 4, inner = H_ * dv_;
        Tensor2 proj(arena.take(static_cast<size_t>(T) * ld * 4), F32, T, N, ld);
        h.linear(in_, proj, STORE_F32, nullptr, arena, s);
        StageTimes::get().mark("in_proj", s);
        // queries and keys lie side by side: one turn over 2 * heads heads
        if (rot_dims_ > 0) rotary_rows(proj, 0, 2 * H_, d_, rot_dims_, rot_base_, step.positions, s);
        Tensor2 decay;
        if (rank_ > 0) {
            decay = arena.tensor(F32, T, H_ * d_);
            lowrank_decay(proj, a_col_, decay_map_, decay_bias_, tau_, decay, s);
        }
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
        decay_scan(proj, 0, k_col_, v_col_, rank_ > 0 ? &decay : nullptr, head_decay_, q_scale_, k_scale_, st, 0, H_, d_, dv_, y, ws, ws_floats, s);
        StageTimes::get().mark("scan", s);
        Tensor2 normed = arena.tensor(dtype_, T, inner);
        rmsnorm_gate_after(y, norm_, eps_, H_, proj, g_col_, normed, s, parts, static_cast<size_t>(T) * inner);
        out_(normed, x, out_epilogue, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * ((in_.out_features() + 4) * 4 + (rank_ > 0 ? H_ * d_ * 4 : 0) + hgrn2_parts(d_) * H_ * dv_ * 4 +
                                              (H_ * dv_ + in_.in_features()) * dtype_size(dtype_)) +
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
        c.weight_bytes += 4.0 * (static_cast<double>(H_) * d_ * (rank_ + 1) + H_ * dv_);
        c.flops_per_token += 4.0 * H_ * d_ * dv_ + 2.0 * H_ * d_ * rank_;          // the state's update and readout, the decays' map
    }

private:
    int H_ = 0, d_ = 0, dv_ = 0, dtype_ = BF16, rot_dims_ = 0, rank_ = 0;
    int k_col_ = 0, v_col_ = 0, g_col_ = 0, a_col_ = 0;
    float eps_ = 1e-6f, q_scale_ = 1.f, k_scale_ = 1.f, tau_ = 1.f;
    double rot_base_ = 10000.0;
    Linear in_, out_;
    Tensor2 decay_map_;
    const float *decay_bias_ = nullptr, *head_decay_ = nullptr, *norm_ = nullptr;
    size_t state_floats_ = 0;
};

// A mixture of small feed-forward experts beside an optional shared one:
//   y = sum_(e chosen) w_e W_down,e act(W_up,e h) + W_down,s act(W_up,s h),   act(z) = relu(z)^2
// The router's logits W_r h are a product of their own with fp32 results (its operands are the compute dtype's: a
// checkpoint's bfloat16 router is held exactly); the scores are their softmax over all experts, or (router "sigmoid")
// every logit's sigmoid on its own, in fp32; the `top` experts with the largest scores are chosen (the lower index
// wins a tie) and w_e = scale * score_e, not renormalised. The experts' first products are one
// joined product (up.weight rows [expert 0 | expert 1 | ... | shared]), the activation multiplies every expert's
// block by w_e (zero for an expert that was not chosen), and the second products are one joined product too
// (down.weight columns in the same order).
// With the activation "clamped_glu" an expert is gated and clamped,
//   expert(h) = W_down (g sigmoid(alpha g) (u + 1)),  g = min(W_gate h, limit),  u = clamp(W_up h, -limit, limit),
// up.weight's rows are [expert 0: gate | up] ... [shared: gate | up] (ff rows each; the shared expert shared_ff, with a
// limit of its own), and with weight_on_input the weight multiplies what the expert READS, y = sum_e expert_e(w_e h):
// the gate's and the up's products are linear, so the activation scales them before it clamps. With shared_gate the
// router's matrix has one more row, and the shared expert's result is multiplied by the sigmoid of that logit.
// Parameters: dtype, experts, ff (an expert's hidden width), top, scale, strings activation, router (softmax);
// clamped_glu: limit, shared_limit, alpha, weight_on_input, shared_gate; tensors router [experts (+ 1), width],
// up.weight [experts * ff + shared_ff (clamped_glu: twice that), width], down.weight [width, experts * ff + shared_ff].
class RoutedExperts final : public FeedForward {
public:
    explicit RoutedExperts(const Params& p) {
        dtype_ = p.integer("dtype");
        glu_.experts = E_ = p.integer("experts"); glu_.ff = ff_ = p.integer("ff"); glu_.top = top_ = p.integer("top");
        glu_.scale = scale_ = static_cast<float>(p.number("scale", 1.0));
        const std::string& act = p.string("activation");
        if (act == "clamped_glu") gated_ = true;
        else if (act != "relu2") fail("routed_experts: unknown activation '%s' (known: relu2, clamped_glu)", act.c_str());
        if (p.str.count("router")) {
            const std::string& r = p.string("router");
            if (r == "sigmoid") glu_.sigmoid_router = true;
            else if (r != "softmax") fail("routed_experts: unknown router '%s' (known: softmax, sigmoid)", r.c_str());
        }
        if (glu_.sigmoid_router && !gated_) fail("routed_experts: sigmoid scores go with the clamped_glu activation");
        up_ = Linear(p.weights("up.weight"), nullptr);
        down_ = Linear(p.weights("down.weight"), nullptr);
        router_ = Linear(p.weights("router"), nullptr);
        if (E_ < 1 || ff_ < 1 || top_ < 1 || top_ > E_) fail("routed_experts: %d of %d experts of %d do not fit", top_, E_, ff_);
        if (gated_) {
            glu_.limit = static_cast<float>(p.number("limit"));
            glu_.alpha = static_cast<float>(p.number("alpha", 1.0));
            glu_.weight_on_input = p.number("weight_on_input", 0) != 0;
            glu_.shared_gate = p.number("shared_gate", 0) != 0;
            glu_.shared_ff = down_.in_features() - E_ * ff_;
            glu_.shared_limit = glu_.shared_ff > 0 ? static_cast<float>(p.number("shared_limit")) : 0.f;
            if (!(glu_.limit > 0.f) || (glu_.shared_ff > 0 && !(glu_.shared_limit > 0.f))) fail("routed_experts: the limits must be positive");
            if (glu_.shared_ff < 0 || up_.out_features() != 2 * down_.in_features() || (glu_.shared_gate && glu_.shared_ff == 0))
                fail("routed_experts: the joined products' shapes do not fit %d gated experts of %d", E_, ff_);
        } else if (up_.out_features() < E_ * ff_ || down_.in_features() != up_.out_features()) {
            fail("routed_experts: the joined products' shapes do not fit %d experts of %d", E_, ff_);
        }
        if (router_.out_features() != E_ + (glu_.shared_gate ? 1 : 0) || router_.in_features() != up_.in_features())
            fail("routed_experts: the router must be [%d, %d]", E_ + (glu_.shared_gate ? 1 : 0), up_.in_features());
        if (down_.out_features() != up_.in_features()) fail("routed_experts: the second products must lead back to the width");
    }
    void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        run(h, step, x, arena, s, ADD_RESIDUAL);
    }
    void forward_set(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        run(h, step, x, arena, s, STORE_F32);
    }
    void run(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s, int out_epilogue) const {
        Pending p;
        first_products(h, step, arena, s, p, false);
        rest(p, step, x, arena, s, out_epilogue);
    }
    bool begin(NormedInput& h, const StepView& step, Arena& arena, hipStream_t s, Pending& pending) const override {
        // (few rows in bfloat16: each of the two products norms its input itself, and no norm kernel runs)
        first_products(h, step, arena, s, pending, dtype_ == BF16 && step.n_tokens <= tuning().ln_fuse_max_rows);
        return true;
    }
    void finish(const Pending& pending, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        rest(pending, step, x, arena, s, ADD_RESIDUAL);
    }
    // pending.a: the router's logits (fp32), pending.b: the experts' joined first product
    void first_products(NormedInput& h, const StepView& step, Arena& arena, hipStream_t s, Pending& p, bool norm_inside) const {
        const int T = step.n_tokens, N = up_.out_features(), R = router_.out_features();
        const int lde = (R + 3) / 4 * 4;
        p.a = Tensor2(arena.take(static_cast<size_t>(T) * lde * 4), F32, T, R, lde);
        p.b = arena.tensor(dtype_, T, N);
        if (norm_inside) {
            h.linear(router_, p.a, STORE_F32, nullptr, arena, s);
            StageTimes::get().mark("router", s);
            h.linear(up_, p.b, STORE, nullptr, arena, s);
        } else {
            const Tensor2& in = h.tensor(arena, s);
            router_(in, p.a, STORE_F32, nullptr, s);
            StageTimes::get().mark("router", s);
            up_(in, p.b, STORE, nullptr, s);
        }
        StageTimes::get().mark("fc1", s);
    }
    void rest(const Pending& p, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s, int out_epilogue) const {
        if (gated_) {
            Tensor2 act = arena.tensor(dtype_, step.n_tokens, down_.in_features());
            moe_glu_act(p.b, p.a, glu_, act, s);
            down_(act, x, out_epilogue, nullptr, s);
        } else {
            moe_act(p.b, p.a, ff_, top_, scale_, p.b, nullptr, s);            // in place
            down_(p.b, x, out_epilogue, nullptr, s);
        }
        StageTimes::get().mark("fc2", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * ((up_.out_features() + down_.in_features() + up_.in_features()) * dtype_size(dtype_) + (E_ + 8) * 4) + 2048;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override {
        up_.add_cost(c);
        down_.add_cost(c);
        router_.add_cost(c);
    }

private:
    int dtype_ = BF16, E_ = 0, ff_ = 0, top_ = 0;
    float scale_ = 1.f;
    bool gated_ = false;
    MoeGlu glu_;
    Linear up_, down_, router_;
};

// What a layer hands on is a weighted sum of the embedding's output and the results of all layers so far: behind the
// layer of pass p (counted from 0), with X_0 the embedding's output and X_(j+1) the stream as the layer of pass j left
// it, x <- sum_(j <= p + 1) w_p[j] X_j. The streams X_j are kept for the step. Parameters: passes; tensors w0, w1, ...
// (w<p>: p + 2 floats).
class DepthMix final : public StreamStep {
public:
    explicit DepthMix(const Params& p) {
        const int n = p.integer("passes");
        if (n < 1) fail("depth_mix: at least one pass is needed");
        for (int k = 0; k < n; ++k) weights_.push_back(f32_vector(p, ("w" + std::to_string(k)).c_str(), k + 2, "depth_mix"));
    }
    void forward(const Tensor2& x, const Tensor2& kept, int pass, const StepView&, Arena&, hipStream_t s) const override {
        if (pass < 0 || pass >= static_cast<int>(weights_.size())) fail("depth_mix: pass %d of %zu", pass, weights_.size());
        if (kept.data == nullptr || kept.rows < x.rows * (pass + 2)) fail("depth_mix needs room for %d kept streams beside the embedding's output", pass + 1);
        depth_mix(x, kept, pass + 1, weights_[pass], s);
    }
    size_t workspace_bytes(int) const override { return 0; }
    bool wants_embedding_output() const override { return true; }
    int kept_streams() const override { return static_cast<int>(weights_.size()); }
    void add_cost(StepCost& c) const override { c.weight_bytes += 4.0 * (weights_.size() + 1); }

private:
    std::vector<const float*> weights_;
};

}  // namespace

void register_linear_attention_parts() {
    register_mixer("linear_attention", [](const Params& p) { return std::unique_ptr<Mixer>(new LinearAttention(p)); });
    register_feed_forward("routed_experts", [](const Params& p) { return std::unique_ptr<FeedForward>(new RoutedExperts(p)); });
    register_stream_step("depth_mix", [](const Params& p) { return std::unique_ptr<StreamStep>(new DepthMix(p)); });
}

}  // namespace minillm
