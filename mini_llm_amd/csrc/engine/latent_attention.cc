// The latent-attention mixer: queries through a latent, keys and values expanded per head from one cached
// latent row per token, one rotated key part shared by the heads.
#include "parts.h"

namespace minillm {

namespace {

const float* f32_vector(const Params& p, const char* key, int n) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n || !t.contiguous()) fail("latent_attention: '%s' must be contiguous float32 [%d]", key, n);
    return static_cast<const float*>(t.data);
}

// With h the mixer's input, per token:
//   c_q = rmsnorm(W_dq h) * w_dqn;   q = W_uq c_q, per head [plain_dim | rot_dim]
//   W_dkv h = [kv_rank | rot_dim]:  c = rmsnorm(first part) * w_dkvn,  k_rot = the second part, turned
//   per head: k = W_uk c, v = W_uv c;  score = scale * (q_plain . k + turned(q_rot) . k_rot), causal within
//   `window` (0: none), softmax;  out = W_o concat_heads(sum_j p_j v_j), added into the stream.
// The pages hold rows [c | k_rot] and nothing per head (in bfloat16 also c once more, transposed page by page,
// the operand shape of the matrix-core kernel for prompt portions). The kernels work in the latent's space
// (kernels/latent_attention.hip): the plain part of a query is multiplied by W_uk^T first, attention runs
// over the page rows with the first kv_rank columns as values, and W_uv expands the result.
// A mixer without the tensor "dkv.weight" reads pages that another layer's call has written (its execution
// order entry names that cache, write = false) with its own expansions, queries and window.
// The turn is the interleaved one: the pair (2i, 2i+1) of the first rot_dims rotated columns at position p
// by the angle p * rot_base^(-2i / rot_dims).
// Parameters: heads, plain_dim, rot_dim, value_dim, kv_rank, q_rank, window, scale, rot_base, rot_dims, eps,
// dtype; tensors dq.weight, dq.norm, uq.weight, [dkv.weight, dkv.norm,] uk.weight (transposed: [kv_rank,
// heads * plain_dim], the layout in which queries are carried into the latent's space), uv.weight, out.weight.
class LatentAttention final : public Mixer {
public:
    explicit LatentAttention(const Params& p) {
        sh_.n_heads = p.integer("heads");
        sh_.plain_dim = p.integer("plain_dim");
        sh_.rot_dim = p.integer("rot_dim");
        sh_.value_dim = p.integer("value_dim");
        sh_.kv_rank = p.integer("kv_rank");
        sh_.q_rank = p.integer("q_rank");
        sh_.rot_dims = p.integer("rot_dims");
        sh_.rot_base = p.number("rot_base");
        sh_.eps = static_cast<float>(p.number("eps"));
        window_ = static_cast<int>(p.number("window", 0));
        scale_ = static_cast<float>(p.number("scale"));
        dtype_ = p.integer("dtype");
        if (sh_.n_heads < 1 || sh_.plain_dim < 1 || sh_.rot_dim < 0 || sh_.value_dim < 1 || sh_.kv_rank < 1 || sh_.q_rank < 1 || window_ < 0)
            fail("latent_attention: heads and sizes must be positive");
        if (sh_.rot_dim % 2 != 0 || sh_.rot_dims % 2 != 0 || sh_.rot_dims > sh_.rot_dim || sh_.rot_dims < 0)
            fail("latent_attention: %d of %d rotated columns: both must be even, the first at most the second", sh_.rot_dims, sh_.rot_dim);
        const int qd = sh_.n_heads * (sh_.plain_dim + sh_.rot_dim);
        dq_ = Linear(p.weights("dq.weight"), nullptr);
        uq_ = Linear(p.weights("uq.weight"), nullptr);
        out_ = Linear(p.weights("out.weight"), nullptr);
        uk_ = p.weights("uk.weight");
        uv_ = p.weights("uv.weight");
        if (dq_.out_features() != sh_.q_rank || uq_.in_features() != sh_.q_rank || uq_.out_features() != qd)
            fail("latent_attention: the query projections do not fit %d heads of %d + %d through %d", sh_.n_heads, sh_.plain_dim, sh_.rot_dim, sh_.q_rank);
        if (uk_.cols != static_cast<int64_t>(sh_.n_heads) * sh_.plain_dim || uk_.rows != sh_.kv_rank || uv_.rows != static_cast<int64_t>(sh_.n_heads) * sh_.value_dim ||
            uv_.cols != sh_.kv_rank || uk_.dtype != dtype_ || uv_.dtype != dtype_)
            fail("latent_attention: the key/value expansions do not fit %d heads and a latent of %d", sh_.n_heads, sh_.kv_rank);
        if (out_.in_features() != sh_.n_heads * sh_.value_dim) fail("latent_attention: the out-projection does not take %d heads of %d", sh_.n_heads, sh_.value_dim);
        dq_norm_ = f32_vector(p, "dq.norm", sh_.q_rank);
        if (p.weights_or_null("dkv.weight") != nullptr) {
            dkv_ = Linear(p.weights("dkv.weight"), nullptr);
            if (dkv_.out_features() != sh_.kv_rank + sh_.rot_dim || dkv_.in_features() != dq_.in_features())
                fail("latent_attention: the key/value latent's projection must have %d rows", sh_.kv_rank + sh_.rot_dim);
            dkv_norm_ = f32_vector(p, "dkv.norm", sh_.kv_rank);
            own_kv_ = true;
        }
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        const int E = sh_.kv_rank + sh_.rot_dim, T = step.n_tokens, g = cache.group, H = sh_.n_heads;
        if (!cache.has_pages() || cache.k_pages.cols != E) fail("latent_attention needs pages of %d-wide rows", E);
        if (write && !own_kv_) fail("a latent-attention layer without a key/value latent of its own cannot write a cache");
        Tensor2 dq = arena.tensor(F32, T, sh_.q_rank), cq = arena.tensor(dtype_, T, sh_.q_rank);
        const bool fill = own_kv_ && write;
        Tensor2 dkv;
        if (fill) dkv = arena.tensor(F32, T, E);
        if (T <= tuning().ln_fuse_max_rows) {
            // few rows: each product normalises the mixer's input itself, and no norm kernel runs
            h.linear(dq_, dq, STORE_F32, nullptr, arena, s);
            if (fill) h.linear(dkv_, dkv, STORE_F32, nullptr, arena, s);
        } else {
            const Tensor2& in = h.tensor(arena, s);
            dq_(in, dq, STORE_F32, nullptr, s);
            if (fill) dkv_(in, dkv, STORE_F32, nullptr, s);
        }
        LatentPages pages;
        pages.rows = cache.k_pages; pages.latent_t = cache.v_pages; pages.page_size = cache.page_size;
        latent_prepare(dq, dq_norm_, cq, fill ? &dkv : nullptr, dkv_norm_, fill ? &pages : nullptr, step.slots[g], step.positions, sh_, s);
        Tensor2 q = arena.tensor(dtype_, T, H * (sh_.plain_dim + sh_.rot_dim));
        uq_(cq, q, STORE, nullptr, s);
        Tensor2 qa = arena.tensor(dtype_, T, H * E);
        latent_absorb(q, uk_, qa, step.positions, sh_, s);
        StageTimes::get().mark("qkv", s);
        Tensor2 o_lat = arena.tensor(dtype_, T, H * sh_.kv_rank);
        LatentStep ls;
        ls.block_tables = step.block_tables[g]; ls.max_blocks = step.max_blocks[g]; ls.n_seqs = step.n_seqs; ls.max_q_len = step.max_q_len;
        ls.token_seq = step.token_seq; ls.positions = step.positions; ls.cu_q = step.cu_q; ls.ctx_len = step.ctx_len;
        ls.max_ctx_len = step.max_ctx_len;
        // (room for the states of split keys, used by steps of few rows only)
        const size_t ws_floats = dtype_ == BF16 ? latent_attention_workspace_floats(sh_.kv_rank) : 0;
        float* ws = ws_floats ? static_cast<float*>(arena.take(ws_floats * 4)) : nullptr;
        latent_attention(qa, pages, ls, scale_, window_, sh_, o_lat, ws, ws_floats, s);
        StageTimes::get().mark("attention", s);
        Tensor2 o = arena.tensor(dtype_, T, H * sh_.value_dim);
        latent_expand(o_lat, uv_, o, sh_, s);
        out_(o, x, ADD_RESIDUAL, nullptr, s);
        StageTimes::get().mark("out_proj", s);
    }
    size_t workspace_bytes(int tokens) const override {
        const size_t E = sh_.kv_rank + sh_.rot_dim, H = sh_.n_heads;
        const size_t per_token = (sh_.q_rank + E) * 4 + (dq_.in_features() + sh_.q_rank + H * (sh_.plain_dim + sh_.rot_dim) + H * E + H * sh_.kv_rank + H * sh_.value_dim) * dtype_size(dtype_);
        return static_cast<size_t>(tokens) * per_token + (dtype_ == BF16 ? latent_attention_workspace_floats(sh_.kv_rank) * 4 : 0) + 8192;
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        // (the "value" pool holds the latent once more, transposed page by page, for the matrix-core kernel:
        // only the bfloat16 path has that kernel)
        n.kind = 1; n.n_kv_heads = 1; n.head_dim = sh_.kv_rank + sh_.rot_dim; n.value_dim = dtype_ == BF16 ? sh_.kv_rank : 0; n.window = window_;
        return n;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override {
        dq_.add_cost(c); uq_.add_cost(c); out_.add_cost(c);
        if (own_kv_) dkv_.add_cost(c);
        c.weight_bytes += static_cast<double>(uk_.cols + uv_.rows) * sh_.kv_rank * dtype_size(dtype_);
        c.flops_per_token += 2.0 * (uk_.cols + uv_.rows) * sh_.kv_rank;
        c.attention_flops_per_key += 2.0 * sh_.n_heads * (2.0 * sh_.kv_rank + sh_.rot_dim);
    }

private:
    LatentShape sh_;
    int window_ = 0, dtype_ = BF16;
    float scale_ = 1.f;
    bool own_kv_ = false;
    Linear dq_, uq_, dkv_, out_;
    Tensor2 uk_, uv_;
    const float *dq_norm_ = nullptr, *dkv_norm_ = nullptr;
};

}  // namespace

void register_latent_attention() {
    register_mixer("latent_attention", [](const Params& p) { return std::unique_ptr<Mixer>(new LatentAttention(p)); });
}

}  // namespace minillm
