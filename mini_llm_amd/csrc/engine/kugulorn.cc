// Kugulorn: a decoder whose configuration lists its layers one by one. A layer has a mixer (latent attention
// or Mamba-2) and optionally a clamped gated feed-forward, each between an RMS norm in front and one behind,
// with a per-column layer scale and one residual multiplier; an untied head behind a final RMS norm; no
// position table (latent attention turns its rotated parts itself). This file reads the configuration, names
// the tensors and chooses the parts; the mechanisms are the parts' own.
//
// config.json: {"architecture": "Kugulorn", "vocab", "width", "residual_mult", "norm": {"eps"},
//   "layers": [{"type": "mamba2", "mixer": {"heads", "vdim", "state", "groups", "conv", "norm_groups"}, "mlp": null},
//              {"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale",
//                "mask": {"size"}, "rot": {"base", "dims"}, ["kv_from": j]}, "mlp": {"kind": "dense", "ff", "limit"}}, ...]}
// Tensors: embed, l<i>.norm1/norm1b[/norm2/norm2b], l<i>.ls1[/ls2], l<i>.mix.*, l<i>.mlp.gate/up/down,
// final.norm, head; linear weights are stored [out, in].
#include <cmath>

#include "arch.h"

namespace minillm {

namespace {

// The design fixes the gate's slope in the feed-forward: y = g sigmoid(1.702 g) (u + 1).
constexpr double GATE_SLOPE = 1.702;

int64_t need_int(const Json& c, const char* key, const std::string& where, int64_t least = 1) {
    const Json* v = c.find(key);
    if (v == nullptr || !v->is_integer()) throw ConfigError("config.json: " + where + "integer key '" + key + "' is missing");
    if (v->integer() < least) throw ConfigError("config.json: " + where + "'" + key + "' must be at least " + std::to_string(least));
    return v->integer();
}
double need_num(const Json& c, const char* key, const std::string& where) {
    const Json* v = c.find(key);
    if (v == nullptr || !v->is_number()) throw ConfigError("config.json: " + where + "number key '" + key + "' is missing");
    return v->number();
}
const Json& need_object(const Json& c, const char* key, const std::string& where) {
    const Json* v = c.find(key);
    if (v == nullptr || !v->is_object()) throw ConfigError("config.json: " + where + "object '" + key + "' is missing");
    return *v;
}

struct LayerConfig {
    enum Kind { Mamba2, LatentAttention } kind = Mamba2;
    // mamba2
    int64_t heads = 0, vdim = 0, state = 0, groups = 0, conv = 0, norm_groups = 1;
    // latent attention
    int64_t dim = 0, rot_dim = 0, kv_rank = 0, q_rank = 0, window = 0, rot_dims = 0, kv_from = -1;
    double scale = 1.0, rot_base = 10000.0;
    // feed-forward
    bool has_mlp = false;
    int64_t ff = 0;
    double limit = 0.0;
};

struct KugulornConfig {
    int64_t vocab = 0, width = 0;
    double eps = 1e-6, residual_mult = 1.0;
    std::vector<LayerConfig> layers;

    explicit KugulornConfig(const Json& c) {
        vocab = need_int(c, "vocab", "");
        width = need_int(c, "width", "");
        residual_mult = need_num(c, "residual_mult", "");
        eps = need_num(need_object(c, "norm", ""), "eps", "norm: ");
        if (!(eps > 0)) throw ConfigError("config.json: norm.eps must be positive");
        const Json* ls = c.find("layers");
        if (ls == nullptr || !ls->is_array() || ls->array().empty()) throw ConfigError("config.json: 'layers' must be a list of layers");
        for (size_t i = 0; i < ls->array().size(); ++i) {
            const Json& l = ls->array()[i];
            const std::string where = "layer " + std::to_string(i) + ": ";
            if (!l.is_object()) throw ConfigError("config.json: " + where + "not an object");
            const Json* type = l.find("type");
            if (type == nullptr || !type->is_string()) throw ConfigError("config.json: " + where + "'type' is missing");
            const Json& m = need_object(l, "mixer", where);
            LayerConfig lc;
            if (type->string() == "mamba2") {
                lc.kind = LayerConfig::Mamba2;
                lc.heads = need_int(m, "heads", where); lc.vdim = need_int(m, "vdim", where); lc.state = need_int(m, "state", where);
                lc.groups = need_int(m, "groups", where); lc.conv = need_int(m, "conv", where); lc.norm_groups = need_int(m, "norm_groups", where);
                if (lc.heads % lc.groups != 0) throw ConfigError("config.json: " + where + "heads is not a multiple of groups");
                if ((lc.heads * lc.vdim) % lc.norm_groups != 0) throw ConfigError("config.json: " + where + "heads * vdim is not a multiple of norm_groups");
                if (lc.conv > 16) throw ConfigError("config.json: " + where + "a convolution of more than 16 taps is not supported");
            } else if (type->string() == "latent_attention") {
                lc.kind = LayerConfig::LatentAttention;
                lc.heads = need_int(m, "heads", where); lc.dim = need_int(m, "dim", where); lc.rot_dim = need_int(m, "rot_dim", where, 0);
                lc.vdim = need_int(m, "vdim", where); lc.kv_rank = need_int(m, "kv_rank", where); lc.q_rank = need_int(m, "q_rank", where);
                lc.scale = need_num(m, "scale", where);
                lc.window = need_int(need_object(m, "mask", where), "size", where + "mask: ");
                if (lc.rot_dim > 0) {
                    const Json& rot = need_object(m, "rot", where);
                    lc.rot_base = need_num(rot, "base", where + "rot: ");
                    lc.rot_dims = need_int(rot, "dims", where + "rot: ", 0);
                    if (!(lc.rot_base > 0)) throw ConfigError("config.json: " + where + "rot.base must be positive");
                }
                if (lc.rot_dims % 2 != 0 || lc.rot_dim % 2 != 0 || lc.rot_dims > lc.rot_dim)
                    throw ConfigError("config.json: " + where + "rot.dims and rot_dim must be even, rot.dims at most rot_dim");
                if (const Json* from = m.find("kv_from")) {
                    if (!from->is_null()) {
                        if (!from->is_integer() || from->integer() < 0 || from->integer() >= static_cast<int64_t>(i))
                            throw ConfigError("config.json: " + where + "kv_from must name an earlier layer");
                        lc.kv_from = from->integer();
                        const LayerConfig& src = layers[static_cast<size_t>(lc.kv_from)];
                        if (src.kind != LayerConfig::LatentAttention || src.kv_from >= 0)
                            throw ConfigError("config.json: " + where + "kv_from must name a latent-attention layer with a key/value latent of its own");
                        if (src.kv_rank != lc.kv_rank || src.rot_dim != lc.rot_dim || src.rot_dims != lc.rot_dims || src.rot_base != lc.rot_base)
                            throw ConfigError("config.json: " + where + "kv_rank, rot_dim and the rotation must equal those of the layer kv_from names");
                    }
                }
            } else {
                throw ConfigError("config.json: " + where + "unknown layer type '" + type->string() + "' (known: latent_attention, mamba2)");
            }
            const Json* mlp = l.find("mlp");
            if (mlp != nullptr && !mlp->is_null()) {
                if (!mlp->is_object()) throw ConfigError("config.json: " + where + "'mlp' must be an object or null");
                const Json* kind = mlp->find("kind");
                if (kind == nullptr || !kind->is_string() || kind->string() != "dense")
                    throw ConfigError("config.json: " + where + "mlp.kind must be 'dense'");
                lc.has_mlp = true;
                lc.ff = need_int(*mlp, "ff", where + "mlp: ");
                lc.limit = need_num(*mlp, "limit", where + "mlp: ");
                if (!(lc.limit > 0)) throw ConfigError("config.json: " + where + "mlp.limit must be positive");
            }
            layers.push_back(lc);
        }
    }
};

std::vector<ParamSpec> kugulorn_specs(const Json& config) {
    const KugulornConfig c(config);
    const int64_t D = c.width;
    std::vector<ParamSpec> s;
    auto matrix = [&](const std::string& n, int64_t r, int64_t k) { s.push_back({n, {r, k}, ParamSpec::Matrix, false, 0.0, 1.0 / std::sqrt(static_cast<double>(k))}); };
    auto vector = [&](const std::string& n, int64_t k, double mean, double std) { s.push_back({n, {k}, ParamSpec::Vector, false, mean, std}); };
    s.push_back({"embed", {c.vocab, D}, ParamSpec::Matrix, false, 0.0, 1.0});
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        vector(L + "norm1", D, 1.0, 0.1);
        vector(L + "norm1b", D, 1.0, 0.1);
        vector(L + "ls1", D, 1.0, 0.2);
        if (l.kind == LayerConfig::Mamba2) {
            const int64_t inner = l.heads * l.vdim, ch = inner + 2 * l.groups * l.state;
            matrix(M + "in", 2 * inner + 2 * l.groups * l.state + l.heads, D);
            s.push_back({M + "conv", {ch, l.conv}, ParamSpec::Vector, false, 0.0, 1.0 / std::sqrt(static_cast<double>(l.conv))});
            vector(M + "conv.b", ch, 0.0, 0.1);
            vector(M + "dt_bias", l.heads, -1.0, 1.0);
            vector(M + "A_log", l.heads, -0.5, 0.7);
            vector(M + "D", l.heads, 1.0, 0.3);
            vector(M + "norm", inner, 1.0, 0.1);
            matrix(M + "o", D, inner);
        } else {
            matrix(M + "dq", l.q_rank, D);
            vector(M + "dq.norm", l.q_rank, 1.0, 0.1);
            matrix(M + "uq", l.heads * (l.dim + l.rot_dim), l.q_rank);
            if (l.kv_from < 0) {
                matrix(M + "dkv", l.kv_rank + l.rot_dim, D);
                vector(M + "dkv.norm", l.kv_rank, 1.0, 0.1);
            }
            // (kept transposed, [kv_rank, heads * dim]: queries are multiplied by it, not the latent)
            s.push_back({M + "uk", {l.heads * l.dim, l.kv_rank}, ParamSpec::Matrix, true, 0.0, 1.0 / std::sqrt(static_cast<double>(l.kv_rank))});
            matrix(M + "uv", l.heads * l.vdim, l.kv_rank);
            matrix(M + "o", D, l.heads * l.vdim);
        }
        if (l.has_mlp) {
            vector(L + "norm2", D, 1.0, 0.1);
            vector(L + "norm2b", D, 1.0, 0.1);
            vector(L + "ls2", D, 1.0, 0.2);
            matrix(L + "mlp.gate", l.ff, D);
            matrix(L + "mlp.up", l.ff, D);
            matrix(L + "mlp.down", D, l.ff);
        }
    }
    vector("final.norm", D, 1.0, 0.1);
    matrix("head", c.vocab, D);
    return s;
}

void kugulorn_assemble(const Json& config, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const KugulornConfig c(config);
    const int D = static_cast<int>(c.width);
    DecoderModel& m = out.model;
    {
        Params e, h;
        e.tensor["table"] = t.at("embed");
        m.embedding = build_embedding("token_table", e);
        h.tensor["weight"] = t.at("head");
        h.num["dtype"] = dtype;
        m.head = build_head("linear", h);
    }
    auto norm = [&](const std::string& name) {
        Params p;
        p.num["size"] = D; p.num["eps"] = c.eps; p.num["dtype"] = dtype;
        p.tensor["weight"] = t.at(name);
        return build_norm("rmsnorm", p);
    };
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        Params a;
        a.num["dtype"] = dtype; a.num["eps"] = c.eps;
        std::unique_ptr<Mixer> mixer;
        if (l.kind == LayerConfig::Mamba2) {
            a.num["heads"] = static_cast<double>(l.heads); a.num["head_dim"] = static_cast<double>(l.vdim); a.num["state"] = static_cast<double>(l.state);
            a.num["groups"] = static_cast<double>(l.groups); a.num["norm_groups"] = static_cast<double>(l.norm_groups);
            a.tensor["in.weight"] = t.at(M + "in"); a.tensor["conv.weight"] = t.at(M + "conv"); a.tensor["conv.bias"] = t.at(M + "conv.b");
            a.tensor["dt_bias"] = t.at(M + "dt_bias"); a.tensor["A_log"] = t.at(M + "A_log"); a.tensor["D"] = t.at(M + "D");
            a.tensor["norm.weight"] = t.at(M + "norm"); a.tensor["out.weight"] = t.at(M + "o");
            mixer = build_mixer("mamba2", a);
        } else {
            a.num["heads"] = static_cast<double>(l.heads); a.num["plain_dim"] = static_cast<double>(l.dim); a.num["rot_dim"] = static_cast<double>(l.rot_dim);
            a.num["value_dim"] = static_cast<double>(l.vdim); a.num["kv_rank"] = static_cast<double>(l.kv_rank); a.num["q_rank"] = static_cast<double>(l.q_rank);
            a.num["window"] = static_cast<double>(l.window); a.num["scale"] = l.scale; a.num["rot_base"] = l.rot_base;
            a.num["rot_dims"] = static_cast<double>(l.rot_dims);
            a.tensor["dq.weight"] = t.at(M + "dq"); a.tensor["dq.norm"] = t.at(M + "dq.norm"); a.tensor["uq.weight"] = t.at(M + "uq");
            if (l.kv_from < 0) { a.tensor["dkv.weight"] = t.at(M + "dkv"); a.tensor["dkv.norm"] = t.at(M + "dkv.norm"); }
            a.tensor["uk.weight"] = t.at(M + "uk"); a.tensor["uv.weight"] = t.at(M + "uv"); a.tensor["out.weight"] = t.at(M + "o");
            mixer = build_mixer("latent_attention", a);
        }
        std::unique_ptr<FeedForward> ff;
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(norm(L + "norm1"));
        norms.push_back(norm(L + "norm1b"));
        Params b;
        b.num["size"] = D; b.num["residual_mult"] = c.residual_mult;
        b.tensor["scale1"] = t.at(L + "ls1");
        if (l.has_mlp) {
            Params f;
            f.num["dtype"] = dtype; f.num["limit"] = l.limit; f.num["alpha"] = GATE_SLOPE;
            f.tensor["gate.weight"] = t.at(L + "mlp.gate"); f.tensor["up.weight"] = t.at(L + "mlp.up"); f.tensor["down.weight"] = t.at(L + "mlp.down");
            ff = build_feed_forward("clamped_gated_mlp", f);
            norms.push_back(norm(L + "norm2"));
            norms.push_back(norm(L + "norm2b"));
            b.tensor["scale2"] = t.at(L + "ls2");
        }
        m.layers.push_back(build_block("sandwich_norm", std::move(mixer), std::move(ff), std::move(norms), b));
        // a layer's cache carries its own index; a layer that shares another's pages reads that layer's
        const bool shares = l.kind == LayerConfig::LatentAttention && l.kv_from >= 0;
        m.order.push_back({static_cast<int>(i), shares ? static_cast<int>(l.kv_from) : static_cast<int>(i), !shares});
    }
    m.final_norm = norm("final.norm");
    out.max_positions = 0;          // positions are not bounded by a table
    if (const Json* e = config.find("eos_token_id")) if (e->is_integer()) out.eos_token_id = static_cast<int>(e->integer());
}

}  // namespace

void register_kugulorn() {
    Architecture a;
    a.name = "Kugulorn";
    a.param_specs = kugulorn_specs;
    a.assemble = kugulorn_assemble;
    register_architecture(a, "kugulorn");
}

}  // namespace minillm
