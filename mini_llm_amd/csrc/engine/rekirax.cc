// Rekirax: a decoder whose configuration lists its layers one by one and may run a group of them several times.
// The embedding is RMS-normed; a layer is pre-norm (norm weights stored around zero and used as 1 + w), its
// mixer reads the normed stream plus a short causal convolution of it, and it has a gated feed-forward with
// biases or none. A mixer is either softmax attention with per-head normed queries and keys, values that are the
// keys before their norm, softcapped scores, a logarithmic distance bias and a sliding window ("attention"), or
// two mixers side by side ("parallel"): chunked attention with whole-row normed, partly rotated queries and keys
// and a sigmoid output gate, and an HGRN2 recurrence; their outputs are RMS-normed over the width and averaged.
// The layers `loop.start .. loop.stop - 1` run `loop.times` times with the same weights and a cache and state of
// their own per run; before every run the stream and the embedding's output go through one linear map side by
// side and a vector of that run is added. The head is the embedding table behind a final norm. This file reads
// the configuration, names the tensors and chooses the parts; the mechanisms are the parts' own.
//
// config.json: {"architecture": "Rekirax", "vocab", "width", "norm": {"eps"}, "canon": {"taps"},
//   "loop": {"start", "stop", "times"},
//   "layers": [{"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask": {"size"}},
//               "mlp": {"kind": "dense", "ff"} | null},
//              {"type": "parallel", "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"},
//               "rot": {"base", "dims"}}, "right": {"heads", "dim", "vdim"}}, "mlp": ...}, ...]}
// Tensors: embed, embed.norm, loop.in, loop.step, l<i>.norm1[/norm2], l<i>.canon1, l<i>.mix.*, l<i>.mlp.*,
// final.norm; linear weights are stored [out, in].
#include <cmath>

#include "arch.h"

namespace minillm {

namespace {

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

struct AttentionConfig {
    int64_t heads = 0, kv_heads = 0, dim = 0, vdim = 0, mask = 0, rot_dims = 0;
    double scale = 1.0, softcap = 0.0, rot_base = 10000.0;
};
struct RecurrenceConfig {
    int64_t heads = 0, dim = 0, vdim = 0;
};
struct LayerConfig {
    enum Kind { Attention, Parallel } kind = Attention;
    AttentionConfig att;            // the attention mixer, or the left one of a parallel pair
    RecurrenceConfig rec;           // the right one of a parallel pair
    bool has_mlp = false;
    int64_t ff = 0;
};

AttentionConfig read_attention(const Json& m, const std::string& where, bool rotated) {
    AttentionConfig a;
    a.heads = need_int(m, "heads", where); a.kv_heads = need_int(m, "kv_heads", where);
    a.dim = need_int(m, "dim", where); a.vdim = need_int(m, "vdim", where);
    a.scale = need_num(m, "scale", where);
    a.mask = need_int(need_object(m, "mask", where), "size", where + "mask: ");
    if (a.heads % a.kv_heads != 0) throw ConfigError("config.json: " + where + "heads is not a multiple of kv_heads");
    if (const Json* cap = m.find("softcap")) {
        if (!cap->is_null()) {
            if (!cap->is_number() || cap->number() < 0) throw ConfigError("config.json: " + where + "softcap must be a number, not negative");
            a.softcap = cap->number();
        }
    }
    if (rotated) {
        const Json& rot = need_object(m, "rot", where);
        a.rot_base = need_num(rot, "base", where + "rot: ");
        a.rot_dims = need_int(rot, "dims", where + "rot: ", 0);
        if (!(a.rot_base > 0) || a.rot_dims % 2 != 0 || a.rot_dims > a.dim)
            throw ConfigError("config.json: " + where + "rot.base must be positive, rot.dims even and at most dim");
    }
    return a;
}

struct RekiraxConfig {
    int64_t vocab = 0, width = 0, taps = 0;
    double eps = 1e-6;
    bool has_loop = false;
    int64_t loop_start = 0, loop_stop = 0, loop_times = 1;
    std::vector<LayerConfig> layers;

    explicit RekiraxConfig(const Json& c) {
        vocab = need_int(c, "vocab", "");
        width = need_int(c, "width", "");
        eps = need_num(need_object(c, "norm", ""), "eps", "norm: ");
        if (!(eps > 0)) throw ConfigError("config.json: norm.eps must be positive");
        if (const Json* canon = c.find("canon")) {
            if (!canon->is_null()) {
                if (!canon->is_object()) throw ConfigError("config.json: 'canon' must be an object");
                taps = need_int(*canon, "taps", "canon: ");
                if (taps > 16) throw ConfigError("config.json: canon.taps: a convolution of more than 16 taps is not supported");
            }
        }
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
            if (type->string() == "attention") {
                lc.kind = LayerConfig::Attention;
                lc.att = read_attention(m, where, false);
                if (lc.att.vdim != lc.att.dim) throw ConfigError("config.json: " + where + "the values are the keys, so vdim must equal dim");
            } else if (type->string() == "parallel") {
                lc.kind = LayerConfig::Parallel;
                lc.att = read_attention(need_object(m, "left", where), where + "left: ", true);
                const Json& r = need_object(m, "right", where);
                lc.rec.heads = need_int(r, "heads", where + "right: "); lc.rec.dim = need_int(r, "dim", where + "right: ");
                lc.rec.vdim = need_int(r, "vdim", where + "right: ");
            } else {
                throw ConfigError("config.json: " + where + "unknown layer type '" + type->string() + "' (known: attention, parallel)");
            }
            const Json* mlp = l.find("mlp");
            if (mlp != nullptr && !mlp->is_null()) {
                if (!mlp->is_object()) throw ConfigError("config.json: " + where + "'mlp' must be an object or null");
                const Json* kind = mlp->find("kind");
                if (kind == nullptr || !kind->is_string() || kind->string() != "dense")
                    throw ConfigError("config.json: " + where + "mlp.kind must be 'dense'");
                lc.has_mlp = true;
                lc.ff = need_int(*mlp, "ff", where + "mlp: ");
            }
            layers.push_back(lc);
        }
        if (const Json* loop = c.find("loop")) {
            if (!loop->is_null()) {
                if (!loop->is_object()) throw ConfigError("config.json: 'loop' must be an object");
                has_loop = true;
                loop_start = need_int(*loop, "start", "loop: ", 0);
                loop_stop = need_int(*loop, "stop", "loop: ", 0);
                loop_times = need_int(*loop, "times", "loop: ");
                if (loop_start >= loop_stop || loop_stop > static_cast<int64_t>(layers.size()))
                    throw ConfigError("config.json: loop: start < stop <= the number of layers is needed");
            }
        }
    }
};

std::vector<ParamSpec> rekirax_specs(const Json& config) {
    const RekiraxConfig c(config);
    const int64_t D = c.width;
    std::vector<ParamSpec> s;
    auto matrix = [&](const std::string& n, int64_t r, int64_t k) { s.push_back({n, {r, k}, ParamSpec::Matrix, false, 0.0, 1.0 / std::sqrt(static_cast<double>(k))}); };
    auto vector = [&](const std::string& n, int64_t k, double mean, double std) { s.push_back({n, {k}, ParamSpec::Vector, false, mean, std}); };
    // a norm weight stored around zero, used as 1 + w
    auto norm = [&](const std::string& n) { s.push_back({n, {D}, ParamSpec::Vector, false, 0.0, 0.1, 1.0}); };
    s.push_back({"embed", {c.vocab, D}, ParamSpec::Matrix, false, 0.0, 1.0});
    norm("embed.norm");
    if (c.has_loop) {
        matrix("loop.in", D, 2 * D);
        s.push_back({"loop.step", {c.loop_times, D}, ParamSpec::Vector, false, 0.0, 0.1});
    }
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        norm(L + "norm1");
        if (l.has_mlp) norm(L + "norm2");
        const AttentionConfig& a = l.att;
        if (l.kind == LayerConfig::Attention) {
            matrix(M + "q", a.heads * a.dim, D);
            matrix(M + "k", a.kv_heads * a.dim, D);
            vector(M + "q.norm", a.dim, 1.0, 0.1);
            vector(M + "k.norm", a.dim, 1.0, 0.1);
            vector(M + "r1", a.heads, 0.5, 0.1);
            vector(M + "r2", a.heads, 0.6, 0.1);
            matrix(M + "o", D, a.heads * a.vdim);
        } else {
            const RecurrenceConfig& r = l.rec;
            const std::string A = M + "left.", R = M + "right.";
            matrix(A + "q", a.heads * a.dim, D);
            matrix(A + "k", a.kv_heads * a.dim, D);
            matrix(A + "v", a.kv_heads * a.vdim, D);
            vector(A + "q.norm", a.heads * a.dim, 1.0, 0.1);
            vector(A + "k.norm", a.kv_heads * a.dim, 1.0, 0.1);
            matrix(A + "g", a.heads * a.vdim, D);
            matrix(A + "o", D, a.heads * a.vdim);
            matrix(R + "q", r.heads * r.dim, D);
            matrix(R + "f", r.heads * r.dim, D);
            vector(R + "f.b", r.heads * r.dim, 1.0, 0.5);
            vector(R + "lower", r.heads * r.dim, 0.4, 0.08);
            matrix(R + "v", r.heads * r.vdim, D);
            vector(R + "norm", r.vdim, 1.0, 0.1);
            matrix(R + "o", D, r.heads * r.vdim);
            vector(A + "out", D, 1.0, 0.1);
            vector(R + "out", D, 1.0, 0.1);
        }
        if (l.has_mlp) {
            matrix(L + "mlp.gate", l.ff, D);
            vector(L + "mlp.gate.b", l.ff, 0.0, 0.1);
            matrix(L + "mlp.up", l.ff, D);
            vector(L + "mlp.up.b", l.ff, 0.0, 0.1);
            matrix(L + "mlp.down", D, l.ff);
            vector(L + "mlp.down.b", D, 0.0, 0.1);
        }
        if (c.taps > 0) s.push_back({L + "canon1", {D, c.taps}, ParamSpec::Vector, false, 0.0, 0.5 / std::sqrt(static_cast<double>(c.taps))});
    }
    norm("final.norm");
    return s;
}

std::unique_ptr<Mixer> attention_mixer(const AttentionConfig& a, const std::string& M, bool left, double eps, int dtype,
                                       const std::map<std::string, Tensor2>& t, DeviceTensors& store) {
    Params p;
    p.num["heads"] = static_cast<double>(a.heads); p.num["kv_heads"] = static_cast<double>(a.kv_heads);
    p.num["dim"] = static_cast<double>(a.dim); p.num["value_dim"] = static_cast<double>(a.vdim);
    p.num["scale"] = a.scale; p.num["softcap"] = a.softcap; p.num["eps"] = eps; p.num["dtype"] = dtype;
    p.tensor["q.norm"] = t.at(M + "q.norm"); p.tensor["k.norm"] = t.at(M + "k.norm");
    p.tensor["out.weight"] = t.at(M + "o");
    if (left) {
        // chunked, rotated, with values and an output gate of its own; norms over the whole projections
        p.num["chunk"] = static_cast<double>(a.mask); p.num["rot_dims"] = static_cast<double>(a.rot_dims); p.num["rot_base"] = a.rot_base;
        p.num["gated"] = 1;
        p.str["qk_norm"] = "row";
        p.tensor["in.weight"] = store.join_rows({t.at(M + "q"), t.at(M + "k"), t.at(M + "v"), t.at(M + "g")});
    } else {
        // a sliding window, values that are the keys, a distance bias; norms per head
        p.num["window"] = static_cast<double>(a.mask); p.num["values_from_keys"] = 1;
        p.str["qk_norm"] = "head";
        p.tensor["r1"] = t.at(M + "r1"); p.tensor["r2"] = t.at(M + "r2");
        p.tensor["in.weight"] = store.join_rows({t.at(M + "q"), t.at(M + "k")});
    }
    return build_mixer("scored_attention", p);
}

void rekirax_assemble(const Json& config, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const RekiraxConfig c(config);
    const int D = static_cast<int>(c.width);
    DecoderModel& m = out.model;
    {
        Params e, h;
        e.tensor["table"] = t.at("embed");
        e.tensor["norm.weight"] = t.at("embed.norm");
        e.num["eps"] = c.eps;
        m.embedding = build_embedding("normed_token_table", e);
        h.tensor["weight"] = t.at("embed");          // the head is the embedding table
        h.num["dtype"] = dtype;
        m.head = build_head("linear", h);
    }
    auto norm = [&](const std::string& name) {
        Params p;
        p.num["size"] = D; p.num["eps"] = c.eps; p.num["dtype"] = dtype;
        p.tensor["weight"] = t.at(name);
        return build_norm("rmsnorm", p);
    };
    if (c.has_loop) {
        Params p;
        p.num["dtype"] = dtype;
        p.tensor["weight"] = t.at("loop.in");
        p.tensor["steps"] = t.at("loop.step");
        m.stream_steps.push_back(build_stream_step("embedding_mix", p));
    }
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        std::unique_ptr<Mixer> mixer;
        if (l.kind == LayerConfig::Attention) {
            mixer = attention_mixer(l.att, M, false, c.eps, dtype, t, out.store);
        } else {
            const RecurrenceConfig& r = l.rec;
            const std::string R = M + "right.";
            Params rp;
            rp.num["heads"] = static_cast<double>(r.heads); rp.num["dim"] = static_cast<double>(r.dim); rp.num["value_dim"] = static_cast<double>(r.vdim);
            rp.num["eps"] = c.eps; rp.num["dtype"] = dtype;
            rp.tensor["in.weight"] = out.store.join_rows({t.at(R + "q"), t.at(R + "f"), t.at(R + "v")});
            rp.tensor["f.bias"] = t.at(R + "f.b"); rp.tensor["lower"] = t.at(R + "lower");
            rp.tensor["norm.weight"] = out.store.repeat(t.at(R + "norm"), static_cast<int>(r.heads));     // one weight, shared by the heads
            rp.tensor["out.weight"] = t.at(R + "o");
            Params pp;
            pp.num["size"] = D; pp.num["eps"] = c.eps;
            pp.mixers.push_back(std::shared_ptr<const Mixer>(attention_mixer(l.att, M + "left.", true, c.eps, dtype, t, out.store).release()));
            pp.mixers.push_back(std::shared_ptr<const Mixer>(build_mixer("hgrn2", rp).release()));
            pp.tensor["norm0"] = t.at(M + "left.out"); pp.tensor["norm1"] = t.at(R + "out");
            pp.tensor["norms"] = out.store.join_rows({t.at(M + "left.out"), t.at(R + "out")});
            mixer = build_mixer("parallel", pp);
        }
        std::unique_ptr<FeedForward> ff;
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(norm(L + "norm1"));
        if (l.has_mlp) {
            Params f;
            f.num["dtype"] = dtype;
            f.str["activation"] = "gelu_tanh";          // the design fixes the tanh form of GELU
            f.tensor["gate_up.weight"] = out.store.join_rows({t.at(L + "mlp.gate"), t.at(L + "mlp.up")});
            f.tensor["gate_up.bias"] = out.store.join_rows({t.at(L + "mlp.gate.b"), t.at(L + "mlp.up.b")});
            f.tensor["down.weight"] = t.at(L + "mlp.down"); f.tensor["down.bias"] = t.at(L + "mlp.down.b");
            ff = build_feed_forward("gated_mlp", f);
            norms.push_back(norm(L + "norm2"));
        }
        Params b;
        b.num["dtype"] = dtype;
        if (c.taps > 0) b.tensor["mixer_conv"] = t.at(L + "canon1");
        m.layers.push_back(build_block("pre_norm", std::move(mixer), std::move(ff), std::move(norms), b));
    }
    // the order: the layers in front of the loop, the loop's layers once per pass (a cache of its own per run, the
    // stream step in front of each pass's first layer), the layers behind it
    const int n = static_cast<int>(c.layers.size());
    int cache = 0;
    auto call = [&](int layer, int before, int pass) {
        LayerCall lc;
        lc.layer = layer; lc.cache = cache++; lc.write = true; lc.before = before; lc.pass = pass;
        m.order.push_back(lc);
    };
    if (!c.has_loop) {
        for (int i = 0; i < n; ++i) call(i, -1, 0);
    } else {
        for (int i = 0; i < c.loop_start; ++i) call(i, -1, 0);
        for (int pass = 0; pass < c.loop_times; ++pass)
            for (int i = static_cast<int>(c.loop_start); i < c.loop_stop; ++i) call(i, i == c.loop_start ? 0 : -1, pass);
        for (int i = static_cast<int>(c.loop_stop); i < n; ++i) call(i, -1, 0);
    }
    m.final_norm = norm("final.norm");
    out.max_positions = 0;          // positions are not bounded by a table
    if (const Json* e = config.find("eos_token_id")) if (e->is_integer()) out.eos_token_id = static_cast<int>(e->integer());
}

}  // namespace

void register_rekirax() {
    Architecture a;
    a.name = "Rekirax";
    a.param_specs = rekirax_specs;
    a.assemble = rekirax_assemble;
    register_architecture(a, "rekirax");
}

}  // namespace minillm
