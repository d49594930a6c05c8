// The Mamba-2 mixer (state-space duality form: one decay per head and token).
#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int64_t n) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("mamba2: '%s' must be contiguous float32 [%lld]", key, (long long)n);
    return static_cast<const float*>(t.data);
}

// With inner = heads * head_dim, N = state, G = groups, the in-projection's rows are
// [z: inner | x: inner | B: G*N | C: G*N | dt: heads]. x, B and C pass a causal convolution per channel
// (taps [channels, taps], the last tap the current token's) and silu; dt = softplus(dt + dt_bias); per head
// the scan of kernels/ssm.hip; then y * silu(z), an RMS norm in norm_groups equal parts times a weight,
// and the out-projection, added into the stream. Per request the mixer carries the convolution's last
// taps - 1 inputs and the scan's state (fp32) in a state slot. The in-projection's result, the
// convolution, the scan and the norm are fp32 in both precisions; the two projections run in the compute dtype.
// Parameters: heads, head_dim, state, groups, norm_groups, eps, dtype; tensors in.weight, conv.weight,
// conv.bias, dt_bias, A_log, D, norm.weight, out.weight.
class Mamba2Mixer final : public Mixer {
public:
    explicit Mamba2Mixer(const Params& p) {
        H_ = p.integer("heads"); P_ = p.integer("head_dim"); N_ = p.integer("state"); G_ = p.integer("groups");
        norm_groups_ = p.integer("norm_groups");
        eps_ = static_cast<float>(p.number("eps"));
        dtype_ = p.integer("dtype");
        if (H_ < 1 || P_ < 1 || N_ < 1 || G_ < 1 || H_ % G_ != 0) fail("mamba2: %d heads of %d, state %d, %d groups do not fit", H_, P_, N_, G_);
        inner_ = H_ * P_;
        channels_ = inner_ + 2 * G_ * N_;
        if (norm_groups_ < 1 || inner_ % norm_groups_ != 0) fail("mamba2: %d columns do not split into %d norm groups", inner_, norm_groups_);
        in_ = Linear(p.weights("in.weight"), nullptr);
        out_ = Linear(p.weights("out.weight"), nullptr);
        if (in_.out_features() != 2 * inner_ + 2 * G_ * N_ + H_ || out_.in_features() != inner_)
            fail("mamba2: the projections' shapes do not fit %d heads of %d, state %d, %d groups", H_, P_, N_, G_);
        conv_ = p.weights("conv.weight");
        if (conv_.dtype != F32 || conv_.rows != channels_ || !conv_.contiguous() || conv_.cols < 1 || conv_.cols > 16)
            fail("mamba2: the convolution must be contiguous float32 [%d, 1 to 16 taps]", channels_);
        taps_ = static_cast<int>(conv_.cols);
        conv_bias_ = f32_vector(p, "conv.bias", channels_);
        dt_bias_ = f32_vector(p, "dt_bias", H_);
        A_log_ = f32_vector(p, "A_log", H_);
        D_ = f32_vector(p, "D", H_);
        norm_ = f32_vector(p, "norm.weight", inner_);
        carried_floats_ = static_cast<size_t>(taps_ - 1) * channels_;
        slot_floats_ = carried_floats_ + static_cast<size_t>(H_) * P_ * N_;
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        if (!cache.has_state() || cache.state_bytes != slot_floats_ * 4) fail("mamba2 needs a state of %zu floats per request", slot_floats_);
        const int T = step.n_tokens, width = in_.out_features();
        // (rows padded to whole 16 bytes)
        Tensor2 proj(arena.take(static_cast<size_t>(T) * ((width + 3) / 4 * 4) * 4), F32, T, width, (width + 3) / 4 * 4);
        h.linear(in_, proj, STORE_F32, nullptr, arena, s);
        StageTimes::get().mark("in_proj", s);
        StateArgs st;
        st.token_seq = step.token_seq; st.cu_q = step.cu_q; st.state_slots = step.state_slots; st.n_seqs = step.n_seqs;
        st.state = static_cast<float*>(cache.state); st.slot_floats = cache.slot_bytes / 4; st.n_slots = cache.n_slots; st.write = write;
        st.max_q_len = step.max_q_len;
        Tensor2 xbc = arena.tensor(F32, T, channels_);
        conv_silu(proj, inner_, conv_, conv_bias_, st, xbc, s);
        StageTimes::get().mark("conv", s);
        // (the scan leaves its result as shares, one per slice of the state's rows; the norm adds them)
        const int parts = ssm_scan_parts(N_);
        Tensor2 y(arena.take(static_cast<size_t>(parts) * T * inner_ * 4), F32, T, inner_);
        // (portions longer than a chunk are scanned chunk by chunk side by side: room for the chunks' states)
        const size_t ws_floats = step.max_q_len > 64 ? ssm_scan_workspace_floats(T, step.n_seqs, H_, P_, N_) : 0;
        float* ws = ws_floats ? static_cast<float*>(arena.take(ws_floats * 4)) : nullptr;
        ssm_scan(xbc, proj, 2 * inner_ + 2 * G_ * N_, dt_bias_, A_log_, D_, st, carried_floats_, H_, P_, N_, G_, y, ws, ws_floats, s);
        StageTimes::get().mark("scan", s);
        Tensor2 gated = arena.tensor(dtype_, T, inner_);
        const Tensor2 z(proj.data, F32, T, inner_, proj.stride);
        rmsnorm(y, norm_, eps_, norm_groups_, &z, gated, nullptr, s, parts, static_cast<size_t>(T) * inner_);
        out_(gated, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * ((in_.out_features() + 4) * 4 + channels_ * 4 + ssm_scan_parts(N_) * inner_ * 4 + inner_ * dtype_size(dtype_)) +
               ssm_scan_workspace_floats(tokens, 1, H_, P_, N_) * 4 + 8192;
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = 2;
        n.state_bytes = slot_floats_ * 4;
        return n;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override {
        in_.add_cost(c);
        out_.add_cost(c);
        c.weight_bytes += 4.0 * (static_cast<double>(channels_) * (taps_ + 1) + 3.0 * H_ + inner_);
        c.flops_per_token += 2.0 * channels_ * taps_ + 6.0 * inner_ * N_;       // the convolution; the scan's update and readout
    }

private:
    int H_ = 0, P_ = 0, N_ = 0, G_ = 0, norm_groups_ = 1, inner_ = 0, channels_ = 0, taps_ = 0, dtype_ = BF16;
    float eps_ = 1e-6f;
    Linear in_, out_;
    Tensor2 conv_;
    const float *conv_bias_ = nullptr, *dt_bias_ = nullptr, *A_log_ = nullptr, *D_ = nullptr, *norm_ = nullptr;
    size_t carried_floats_ = 0, slot_floats_ = 0;
};

}  // namespace

void register_mamba2() {
    register_mixer("mamba2", [](const Params& p) { return std::unique_ptr<Mixer>(new Mamba2Mixer(p)); });
}

}  // namespace minillm
