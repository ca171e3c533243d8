// RMS norm, the block arrangements with a norm on both sides of each sub-layer, with a norm behind it only, and with
// mixer and feed-forward side by side on one stream, and the clamped gated feed-forward.
#include <algorithm>

#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int n, const char* who) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("%s: '%s' must be contiguous float32 [%d]", who, key, n);
    return static_cast<const float*>(t.data);
}

// h = x / sqrt(mean(x^2) + eps) * weight over the last dimension (eps inside the root), statistics in fp32.
// Parameters: size, eps, dtype, tensor "weight".
class RMSNorm final : public Norm {
public:
    explicit RMSNorm(const Params& p) {
        size_ = p.integer("size");
        eps_ = static_cast<float>(p.number("eps"));
        dtype = p.integer("dtype");
        weight_ = f32_vector(p, "weight", size_, "rmsnorm");
    }
    Tensor2 forward(const Tensor2& x, const int* rows, int n, Arena& arena, hipStream_t s) const override {
        if (x.cols != size_) fail("rmsnorm: rows of %lld, the norm is %d wide", (long long)x.cols, size_);
        Tensor2 h = arena.tensor(dtype, n, size_);
        rmsnorm(x, weight_, eps_, 1, nullptr, h, rows, s);
        return h;
    }
    void forward_into(const Tensor2& x, const int* rows, const Tensor2& out, hipStream_t s) const override {
        if (x.cols != size_) fail("rmsnorm: rows of %lld, the norm is %d wide", (long long)x.cols, size_);
        rmsnorm(x, weight_, eps_, 1, nullptr, out, rows, s);
    }
    bool conv_single(const Tensor2& x, const Tensor2& taps, const StateArgs& st, const Tensor2& out, hipStream_t s) const override {
        if (x.cols != size_) fail("rmsnorm: rows of %lld, the norm is %d wide", (long long)x.cols, size_);
        return rmsnorm_conv_single(x, weight_, eps_, taps, st, out, s);
    }
    bool add_conv_single(const Tensor2& y, const Tensor2& x, const Tensor2& taps, const StateArgs& st, const Tensor2& out,
                         hipStream_t s) const override {
        if (y.cols != size_) fail("rmsnorm: rows of %lld, the norm is %d wide", (long long)y.cols, size_);
        return stream_conv_single(x, &y, weight_, eps_, taps, st, out, s);
    }
    void linear(const Tensor2& x, const Linear& lin, const Tensor2& out, int epilogue, const int* rows,
                const KvScatter* kv, Arena& arena, hipStream_t s) const override {
        if (kv != nullptr) { Norm::linear(x, lin, out, epilogue, rows, kv, arena, s); return; }
        // the norm inside the product where the kernels allow it; otherwise the rows pass through the arena
        const size_t mark = arena.mark();
        void* tmp = arena.take(static_cast<size_t>(out.rows) * size_ * dtype_size(lin.weight.dtype));
        rms_linear(x, weight_, eps_, lin.weight, lin.bias, out, epilogue, rows, tmp, s);
        arena.release(mark);
    }
    void add_scaled(const Tensor2& y, const float* scale, float mult, const Tensor2& x, bool clear, hipStream_t s) const override {
        if (y.cols != size_) fail("rmsnorm: rows of %lld, the norm is %d wide", (long long)y.cols, size_);
        rmsnorm_add(y, weight_, scale, mult, eps_, x, clear, s);
    }
    size_t workspace_bytes(int rows) const override { return static_cast<size_t>(rows) * size_ * dtype_size(dtype) + 256; }
    void add_cost(StepCost& c) const override { c.weight_bytes += 4.0 * size_; }

private:
    int size_ = 0;
    float eps_ = 1e-6f;
    const float* weight_ = nullptr;
};

// A norm in front of and behind each sub-layer, a per-column scale on the sub-layer's normed result and one
// multiplier on what enters the stream:
//   x += mult * scale1 * norm1b(mixer(norm1(x)));   x += mult * scale2 * norm2b(ff(norm2(x)))
// The sub-layer adds its result into a cleared fp32 buffer of the stream's shape; the norm behind it adds
// from there into the stream. Norms: [norm1, norm1b] or [norm1, norm1b, norm2, norm2b]; parameters:
// "size" (the stream's width), "residual_mult" (default 1), tensors "scale1", "scale2" (optional: no scale).
class SandwichNormBlock final : public Block {
public:
    SandwichNormBlock(std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> norms, const Params& p)
        : mixer_(std::move(m)), ff_(std::move(f)) {
        if (!mixer_) fail("a sandwich-norm block needs a mixer");
        if (norms.size() != (ff_ ? 4u : 2u)) fail("a sandwich-norm block has two norms per sub-layer (%d here), got %zu", ff_ ? 4 : 2, norms.size());
        for (auto& n : norms) if (!n) fail("a sandwich-norm block was handed a missing norm");
        pre1_ = std::move(norms[0]);
        post1_ = std::move(norms[1]);
        if (ff_) { pre2_ = std::move(norms[2]); post2_ = std::move(norms[3]); }
        size_ = p.integer("size");
        mult_ = static_cast<float>(p.number("residual_mult", 1.0));
        if (const Tensor2* t = p.weights_or_null("scale1")) scale1_ = checked_scale(*t);
        if (const Tensor2* t = p.weights_or_null("scale2")) scale2_ = checked_scale(*t);
    }
    void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                 hipStream_t s) const override {
        const size_t outer = arena.mark();
        // the sub-layer's result: the step's cleared buffer (left cleared again by the norms behind the
        // sub-layers), or one of this layer's own
        const bool shared = step.zeroed_rows != nullptr;
        Tensor2 y = shared ? Tensor2(step.zeroed_rows, F32, x.rows, x.cols) : arena.tensor(F32, x.rows, x.cols);
        if (!shared) fill_zero(y, s);
        const size_t mark = arena.mark();
        {
            NormedInput h(*pre1_, x);
            mixer_->forward(h, step, cache, y, write, arena, s);
        }
        arena.release(mark);
        if (x.cols != size_) fail("a sandwich-norm block of width %d was handed a stream of %lld", size_, (long long)x.cols);
        post1_->add_scaled(y, static_cast<const float*>(scale1_.data), mult_, x, shared || ff_ != nullptr, s);
        StageTimes::get().mark("post_norm", s);
        if (ff_) {
            {
                NormedInput h(*pre2_, x);
                ff_->forward(h, step, y, arena, s);
            }
            arena.release(mark);
            post2_->add_scaled(y, static_cast<const float*>(scale2_.data), mult_, x, shared, s);
            StageTimes::get().mark("post_norm2", s);
        }
        arena.release(outer);
    }
    size_t workspace_bytes(int tokens) const override {
        size_t a = mixer_->workspace_bytes(tokens) + 2 * pre1_->workspace_bytes(tokens);
        if (ff_) a = std::max(a, ff_->workspace_bytes(tokens) + 2 * pre2_->workspace_bytes(tokens));
        return a + static_cast<size_t>(tokens) * size_ * 4 + 1024;
    }
    CacheNeed cache_need() const override { return mixer_->cache_need(); }
    bool wants_zeroed_rows() const override { return true; }
    void reserve(int max_seqs, hipStream_t s) const override {
        mixer_->reserve(max_seqs, s);
        if (ff_) ff_->reserve(max_seqs, s);
    }
    void add_cost(StepCost& c) const override {
        pre1_->add_cost(c); post1_->add_cost(c);
        mixer_->add_cost(c);
        if (ff_) { pre2_->add_cost(c); post2_->add_cost(c); ff_->add_cost(c); }
        c.weight_bytes += 4.0 * (scale1_.cols + scale2_.cols);
    }

private:
    Tensor2 checked_scale(const Tensor2& t) {
        if (t.dtype != F32 || !t.contiguous() || t.rows * t.cols != size_) fail("a layer scale must be contiguous float32 [%d]", size_);
        return Tensor2(t.data, F32, 1, t.rows * t.cols);
    }
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<FeedForward> ff_;
    std::unique_ptr<Norm> pre1_, post1_, pre2_, post2_;
    Tensor2 scale1_, scale2_;
    float mult_ = 1.f;
    int size_ = 0;               // the stream's width
};


// A norm BEHIND each sub-layer only; the sub-layers read the stream itself:
//   x += norm1(mixer(x));   x += norm2(ff(x))
// With the tensors "mixer_conv" / "ff_conv" ([width, taps] fp32) what a sub-layer reads is x + conv(x): a causal
// convolution over time on each channel, the last tap the token's own; the last taps - 1 rows of each input are carried
// per request in the front of the layer's state slot (the mixer's convolution first, then the feed-forward's; the
// mixer's own state, if it has one, lies behind them). The sub-layer sets an fp32 buffer of the stream's shape and the
// norm adds from there into the stream. Norms: [norm1] or [norm1, norm2]; parameters: dtype, size (the stream's width).
class PostNormBlock final : public Block {
public:
    PostNormBlock(std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> norms, const Params& p)
        : mixer_(std::move(m)), ff_(std::move(f)) {
        if (!mixer_) fail("a post-norm block needs a mixer");
        if (norms.size() != (ff_ ? 2u : 1u)) fail("a post-norm block has one norm per sub-layer (%d here), got %zu", ff_ ? 2 : 1, norms.size());
        for (auto& n : norms) if (!n) fail("a post-norm block was handed a missing norm");
        norm1_ = std::move(norms[0]);
        if (ff_) norm2_ = std::move(norms[1]);
        dtype_ = p.integer("dtype");
        size_ = p.integer("size");
        if (const Tensor2* c = p.weights_or_null("mixer_conv")) conv1_ = checked_conv(*c);
        if (const Tensor2* c = p.weights_or_null("ff_conv")) {
            if (!ff_) fail("a post-norm block without a feed-forward was handed its convolution");
            conv2_ = checked_conv(*c);
        }
        conv1_bytes_ = carried_bytes(conv1_);
        conv2_bytes_ = carried_bytes(conv2_);
    }
    void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                 hipStream_t s) const override {
        const size_t carried = conv1_bytes_ + conv2_bytes_;
        if (carried > 0 && (!cache.has_state() || cache.state_bytes < carried)) fail("a block with input convolutions needs %zu bytes of state per request", carried);
        const size_t outer = arena.mark();
        Tensor2 y = arena.tensor(F32, x.rows, x.cols);       // a sub-layer's result, set by it
        const size_t mark = arena.mark();
        CacheView rest = cache;                              // what lies behind the carried rows is the mixer's
        if (carried > 0) {
            rest.state = static_cast<char*>(cache.state) + carried;
            rest.state_bytes = cache.state_bytes - carried;
            if (rest.state_bytes == 0) rest.kind &= ~2;
        }
        {
            NormedInput h(input(x, conv1_, 0, step, cache, write, arena, s));
            mixer_->forward_set(h, step, rest, y, write, arena, s);
        }
        arena.release(mark);
        // every sequence brings one token: the norm behind the mixer and the feed-forward's convolution in one kernel
        Tensor2 fused;
        if (ff_ && conv2_.data != nullptr && single_tokens(step)) {
            fused = arena.tensor(dtype_, x.rows, x.cols);
            if (!norm1_->add_conv_single(y, x, conv2_, state_args(conv1_bytes_, step, cache, write), fused, s)) {
                fused = Tensor2();
                arena.release(mark);
            }
        }
        if (fused.data == nullptr) norm1_->add_scaled(y, nullptr, 1.f, x, false, s);
        StageTimes::get().mark("post_norm", s);
        if (ff_) {
            {
                NormedInput h(fused.data != nullptr ? fused : input(x, conv2_, conv1_bytes_, step, cache, write, arena, s));
                ff_->forward_set(h, step, y, arena, s);
            }
            arena.release(mark);
            norm2_->add_scaled(y, nullptr, 1.f, x, false, s);
            StageTimes::get().mark("post_norm2", s);
        }
        arena.release(outer);
    }
    size_t workspace_bytes(int tokens) const override {
        size_t a = mixer_->workspace_bytes(tokens);
        if (ff_) a = std::max(a, ff_->workspace_bytes(tokens));
        // the sub-layer's result, and its input in the compute dtype
        return a + static_cast<size_t>(tokens) * size_ * 8 + 2048;
    }
    CacheNeed cache_need() const override {
        CacheNeed n = mixer_->cache_need();
        if (conv1_bytes_ + conv2_bytes_ > 0) { n.kind |= 2; n.state_bytes += conv1_bytes_ + conv2_bytes_; }
        return n;
    }
    void reserve(int max_seqs, hipStream_t s) const override {
        mixer_->reserve(max_seqs, s);
        if (ff_) ff_->reserve(max_seqs, s);
    }
    void add_cost(StepCost& c) const override {
        norm1_->add_cost(c);
        mixer_->add_cost(c);
        if (ff_) { norm2_->add_cost(c); ff_->add_cost(c); }
        for (const Tensor2* t : {&conv1_, &conv2_})
            if (t->data != nullptr) { c.weight_bytes += 4.0 * t->rows * t->cols; c.flops_per_token += 2.0 * t->rows * t->cols; }
    }

private:
    static Tensor2 checked_conv(const Tensor2& c) {
        if (c.dtype != F32 || !c.contiguous() || c.cols < 1 || c.cols > 16) fail("a block's input convolution must be contiguous float32 [width, 1 to 16 taps]");
        return c;
    }
    static size_t carried_bytes(const Tensor2& c) { return c.data ? static_cast<size_t>(c.cols - 1) * c.rows * 4 : 0; }
    // What a sub-layer reads, in the compute dtype: x + conv(x), or x itself.
    Tensor2 input(const Tensor2& x, const Tensor2& conv, size_t state_at, const StepView& step, const CacheView& cache, bool write,
                  Arena& arena, hipStream_t s) const {
        if (conv.data == nullptr) {
            if (dtype_ != F32) fail("a post-norm block without an input convolution runs in float32 only");
            return x;
        }
        if (x.cols != conv.rows) fail("the input convolution has %lld channels, the stream %lld", (long long)conv.rows, (long long)x.cols);
        Tensor2 hc = arena.tensor(dtype_, x.rows, x.cols);
        const StateArgs st = state_args(state_at, step, cache, write);
        // (single tokens: a kernel that asks for all its loads at once)
        if (!(single_tokens(step) && stream_conv_single(x, nullptr, nullptr, 0.f, conv, st, hc, s))) conv_residual(x, conv, st, hc, s);
        StageTimes::get().mark("input_conv", s);
        return hc;
    }
    static bool single_tokens(const StepView& step) { return step.max_q_len == 1 && step.n_tokens == step.n_seqs; }
    // The step's arrays and the carried rows that lie `state_at` bytes into the layer's slot.
    static StateArgs state_args(size_t state_at, const StepView& step, const CacheView& cache, bool write) {
        StateArgs st;
        st.token_seq = step.token_seq; st.cu_q = step.cu_q; st.state_slots = step.state_slots; st.n_seqs = step.n_seqs;
        st.max_q_len = step.max_q_len; st.state = reinterpret_cast<float*>(static_cast<char*>(cache.state) + state_at);
        st.slot_floats = cache.slot_bytes / 4; st.n_slots = cache.n_slots; st.write = write;
        return st;
    }
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<FeedForward> ff_;
    std::unique_ptr<Norm> norm1_, norm2_;
    Tensor2 conv1_, conv2_;           // [width, taps], or empty: no input convolution
    size_t conv1_bytes_ = 0, conv2_bytes_ = 0;
    int dtype_ = BF16, size_ = 0;     // size: the stream's width
};

// Mixer and feed-forward side by side, each behind a norm of its own, both reading the SAME stream:
//   x += mixer(norm1(x)) + ff(norm2(x))
// The feed-forward's input is normed before the mixer adds its result into the stream; then both add theirs. For few
// rows a feed-forward that has halves (FeedForward::begin / finish) runs its first products, with the norm inside
// them, before the mixer and the rest behind it, and no norm kernel runs. Norms: [norm1] or [norm1, norm2].
class ParallelNormBlock final : public Block {
public:
    ParallelNormBlock(std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> norms, const Params&)
        : mixer_(std::move(m)), ff_(std::move(f)) {
        if (!mixer_) fail("a parallel block needs a mixer");
        if (norms.size() != (ff_ ? 2u : 1u)) fail("a parallel block has one norm per sub-layer (%d here), got %zu", ff_ ? 2 : 1, norms.size());
        for (auto& n : norms) if (!n) fail("a parallel block was handed a missing norm");
        norm1_ = std::move(norms[0]);
        if (ff_) norm2_ = std::move(norms[1]);
    }
    void forward(const Tensor2& x, const StepView& step, const CacheView& cache, bool write, Arena& arena,
                 hipStream_t s) const override {
        const size_t outer = arena.mark();
        // Few rows: the feed-forward's first products run before the mixer, with the norm inside them, and the rest
        // behind it; otherwise its input is normed before the mixer changes x.
        Tensor2 h2;
        FeedForward::Pending pending;
        bool halves = false;
        if (ff_ && x.rows <= tuning().ln_fuse_max_rows && x.cols <= tuning().halves_max_width) {
            NormedInput h(*norm2_, x);
            halves = ff_->begin(h, step, arena, s, pending);
        }
        if (ff_ && !halves) h2 = norm2_->forward(x, nullptr, static_cast<int>(x.rows), arena, s);
        const size_t mark = arena.mark();
        {
            NormedInput h(*norm1_, x);
            mixer_->forward(h, step, cache, x, write, arena, s);
        }
        arena.release(mark);
        if (halves) {
            ff_->finish(pending, step, x, arena, s);
        } else if (ff_) {
            NormedInput h(h2);
            ff_->forward(h, step, x, arena, s);
        }
        arena.release(outer);
    }
    size_t workspace_bytes(int tokens) const override {
        // (what the feed-forward's first half leaves in the arena stays there while the mixer runs)
        size_t a = mixer_->workspace_bytes(tokens) + 2 * norm1_->workspace_bytes(tokens);
        if (ff_) a += ff_->workspace_bytes(tokens) + 2 * norm2_->workspace_bytes(tokens);
        return a + 1024;
    }
    CacheNeed cache_need() const override { return mixer_->cache_need(); }
    void reserve(int max_seqs, hipStream_t s) const override {
        mixer_->reserve(max_seqs, s);
        if (ff_) ff_->reserve(max_seqs, s);
    }
    void add_cost(StepCost& c) const override {
        norm1_->add_cost(c);
        mixer_->add_cost(c);
        if (ff_) { norm2_->add_cost(c); ff_->add_cost(c); }
    }

private:
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<FeedForward> ff_;
    std::unique_ptr<Norm> norm1_, norm2_;
};

// y = W_down( g sigmoid(alpha g) (u + 1) ) with g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
// added into the stream it is handed. Parameters: limit, alpha, dtype; tensors gate.weight, up.weight,
// down.weight ([out, in]).
class ClampedGatedMLP final : public FeedForward {
public:
    explicit ClampedGatedMLP(const Params& p) {
        dtype_ = p.integer("dtype");
        limit_ = static_cast<float>(p.number("limit"));
        alpha_ = static_cast<float>(p.number("alpha"));
        if (!(limit_ > 0)) fail("clamped_gated_mlp: the limit must be positive");
        gate_ = Linear(p.weights("gate.weight"), nullptr);
        up_ = Linear(p.weights("up.weight"), nullptr);
        down_ = Linear(p.weights("down.weight"), nullptr);
        if (gate_.out_features() != up_.out_features() || gate_.in_features() != up_.in_features() ||
            down_.in_features() != up_.out_features())
            fail("clamped_gated_mlp: the three products' shapes do not fit");
    }
    void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        const int T = step.n_tokens, F = up_.out_features();
        Tensor2 g = arena.tensor(dtype_, T, F), u = arena.tensor(dtype_, T, F);
        if (T <= tuning().ln_fuse_max_rows) {
            // few rows: each product normalises its input itself, and no norm kernel runs
            h.linear(gate_, g, STORE, nullptr, arena, s);
            h.linear(up_, u, STORE, nullptr, arena, s);
        } else {
            const Tensor2& in = h.tensor(arena, s);
            gate_(in, g, STORE, nullptr, s);
            up_(in, u, STORE, nullptr, s);
        }
        StageTimes::get().mark("fc1", s);
        glu_clamped(g, u, limit_, alpha_, g, s);            // in place over the gate's rows
        down_(g, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("fc2", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * (2 * up_.out_features() + up_.in_features()) * dtype_size(dtype_) + 2048;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override { gate_.add_cost(c); up_.add_cost(c); down_.add_cost(c); }

private:
    int dtype_ = BF16;
    float limit_ = 0.f, alpha_ = 1.f;
    Linear gate_, up_, down_;
};

}  // namespace

void register_gated_parts() {
    register_norm("rmsnorm", [](const Params& p) { return std::unique_ptr<Norm>(new RMSNorm(p)); });
    register_feed_forward("clamped_gated_mlp", [](const Params& p) { return std::unique_ptr<FeedForward>(new ClampedGatedMLP(p)); });
    register_block("sandwich_norm", [](std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> n,
                                       const Params& p) {
        return std::unique_ptr<Block>(new SandwichNormBlock(std::move(m), std::move(f), std::move(n), p));
    });
    register_block("parallel_norm", [](std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> n,
                                       const Params& p) {
        return std::unique_ptr<Block>(new ParallelNormBlock(std::move(m), std::move(f), std::move(n), p));
    });
    register_block("post_norm", [](std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f, std::vector<std::unique_ptr<Norm>> n,
                                   const Params& p) {
        return std::unique_ptr<Block>(new PostNormBlock(std::move(m), std::move(f), std::move(n), p));
    });
}

}  // namespace minillm
