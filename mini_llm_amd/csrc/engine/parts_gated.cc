// RMS norm, the block arrangement with a norm on both sides of each sub-layer, and the clamped gated
// feed-forward.
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
}

}  // namespace minillm
