// Viladra: a decoder whose configuration lists its layers one by one. A sub-layer reads the residual stream itself plus
// a short causal convolution of it over time, and its result is RMS-normed before it is added back (a norm behind
// the sub-layer only). A mixer is linear attention with one fixed decay per head and rotated queries and keys
// ("retention"), linear attention with a decay per key channel from a low-rank map of the input ("gla"), or windowed
// attention whose weights are sigmoids of the scores, with whole-row normed queries and keys, biases, a score bias and
// an output gate per head ("attention"). The feed-forward is a mixture of small squared-ReLU experts beside a shared
// one. What a layer hands on is a learned weighted sum of the embedding's output and the results of all layers so
// far. The embedding is scaled; the head is the embedding table behind a final norm, its logits capped by a tanh.
// This file reads the configuration, names the tensors and chooses the parts; the mechanisms are the parts' own.
//
// config.json: {"architecture": "Viladra", "vocab", "width", "norm": {"eps"}, "canon": {"taps"},
//   "embedding": {"scale"}, "logit_softcap",
//   "layers": [{"type": "retention", "mixer": {"heads", "dim", "vdim", "decay": [..], "rot": {"base", "dims"}}, "mlp": ...},
//              {"type": "gla", "mixer": {"heads", "dim", "vdim", "tau"}, "mlp": ...},
//              {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}}, "mlp": ...}]}
//   mlp: {"kind": "moe", "router": {"experts", "top", "scale"}, "expert": {"ff"}, "shared": {"ff"} | null} | null
//   May be absent: canon, embedding, logit_softcap, rot (none of it), kv_heads (as many as heads), vdim (as wide as dim),
//   mlp.kind, router.scale (1), mlp.shared, mlp.
// Tensors: embed, l<i>.norm1[/norm2], l<i>.canon1[/canon2], l<i>.dwa, l<i>.mix.*, l<i>.mlp.{router, e<k>.up, e<k>.down,
// shared.up, shared.down}, final.norm; linear weights are stored [out, in]. The rank of a gla layer's decay map is
// not in config.json: it is the height of the stored l<i>.mix.a1.
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

struct MixerConfig {
    enum Kind { Retention, Gla, Attention } kind = Retention;
    int64_t heads = 0, kv_heads = 0, dim = 0, vdim = 0, mask = 0, rot_dims = 0, rank = 0;
    double scale = 1.0, rot_base = 10000.0, tau = 1.0;
    std::vector<double> decay;
};
struct MlpConfig {
    bool present = false;
    int64_t experts = 0, top = 0, ff = 0, shared_ff = 0;      // shared_ff 0: no shared expert
    double scale = 1.0;
};
struct LayerConfig {
    MixerConfig mix;
    MlpConfig mlp;
};

// The default rank of a gla layer's decay map, used where no checkpoint says otherwise (random weights).
const int64_t kDefaultDecayRank = 16;

struct ViladraConfig {
    int64_t vocab = 0, width = 0, taps = 0;
    double eps = 1e-6, embed_scale = 1.0, logit_softcap = 0.0;
    std::vector<LayerConfig> layers;

    explicit ViladraConfig(const Json& c) {
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
        if (const Json* e = c.find("embedding")) {
            if (!e->is_null()) {
                if (!e->is_object()) throw ConfigError("config.json: 'embedding' must be an object");
                embed_scale = need_num(*e, "scale", "embedding: ");
            }
        }
        if (const Json* cap = c.find("logit_softcap")) {
            if (!cap->is_null()) {
                if (!cap->is_number() || !(cap->number() > 0)) throw ConfigError("config.json: logit_softcap must be a positive number or null");
                logit_softcap = cap->number();
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
            MixerConfig& x = lc.mix;
            x.heads = need_int(m, "heads", where); x.dim = need_int(m, "dim", where);
            x.vdim = m.find("vdim") != nullptr ? need_int(m, "vdim", where) : x.dim;          // (no vdim: values as wide as keys)
            if (type->string() == "retention") {
                x.kind = MixerConfig::Retention;
                const Json* dec = m.find("decay");
                if (dec == nullptr || !dec->is_array() || static_cast<int64_t>(dec->array().size()) != x.heads)
                    throw ConfigError("config.json: " + where + "'decay' must list one number per head");
                for (const Json& v : dec->array()) {
                    if (!v.is_number() || !(v.number() > 0) || v.number() > 1) throw ConfigError("config.json: " + where + "a decay must lie in (0, 1]");
                    x.decay.push_back(v.number());
                }
                if (const Json* rot = m.find("rot")) {
                    if (!rot->is_null()) {
                        if (!rot->is_object()) throw ConfigError("config.json: " + where + "'rot' must be an object");
                        x.rot_base = need_num(*rot, "base", where + "rot: ");
                        x.rot_dims = need_int(*rot, "dims", where + "rot: ", 0);
                        if (!(x.rot_base > 0) || x.rot_dims % 2 != 0 || x.rot_dims > x.dim)
                            throw ConfigError("config.json: " + where + "rot.base must be positive, rot.dims even and at most dim");
                    }
                }
            } else if (type->string() == "gla") {
                x.kind = MixerConfig::Gla;
                x.tau = need_num(m, "tau", where);
                if (!(x.tau > 0)) throw ConfigError("config.json: " + where + "tau must be positive");
                x.rank = kDefaultDecayRank;
                if (const Json* r = m.find("rank")) if (r->is_integer() && r->integer() >= 1) x.rank = r->integer();
            } else if (type->string() == "attention") {
                x.kind = MixerConfig::Attention;
                x.kv_heads = m.find("kv_heads") != nullptr ? need_int(m, "kv_heads", where) : x.heads;     // (none: no grouping)
                if (x.heads % x.kv_heads != 0) throw ConfigError("config.json: " + where + "heads is not a multiple of kv_heads");
                x.scale = need_num(m, "scale", where);
                x.mask = need_int(need_object(m, "mask", where), "size", where + "mask: ");
            } else {
                throw ConfigError("config.json: " + where + "unknown layer type '" + type->string() + "' (known: retention, gla, attention)");
            }
            const Json* mlp = l.find("mlp");
            if (mlp != nullptr && !mlp->is_null()) {
                if (!mlp->is_object()) throw ConfigError("config.json: " + where + "'mlp' must be an object or null");
                const Json* kind = mlp->find("kind");
                if (kind != nullptr && (!kind->is_string() || kind->string() != "moe"))
                    throw ConfigError("config.json: " + where + "mlp.kind must be 'moe'");
                MlpConfig& f = lc.mlp;
                f.present = true;
                const Json& r = need_object(*mlp, "router", where + "mlp: ");
                f.experts = need_int(r, "experts", where + "mlp: router: ");
                f.top = need_int(r, "top", where + "mlp: router: ");
                if (f.top > f.experts) throw ConfigError("config.json: " + where + "mlp: router.top exceeds router.experts");
                if (f.experts > 256) throw ConfigError("config.json: " + where + "mlp: more than 256 experts are not supported");
                if (const Json* sc = r.find("scale")) {
                    if (!sc->is_number()) throw ConfigError("config.json: " + where + "mlp: router.scale must be a number");
                    f.scale = sc->number();
                }
                f.ff = need_int(need_object(*mlp, "expert", where + "mlp: "), "ff", where + "mlp: expert: ");
                if (const Json* sh = mlp->find("shared")) {
                    if (!sh->is_null()) {
                        if (!sh->is_object()) throw ConfigError("config.json: " + where + "mlp: 'shared' must be an object or null");
                        f.shared_ff = need_int(*sh, "ff", where + "mlp: shared: ");
                    }
                }
            }
            layers.push_back(lc);
        }
    }
};

std::vector<ParamSpec> viladra_specs(const Json& config) {
    const ViladraConfig c(config);
    const int64_t D = c.width;
    std::vector<ParamSpec> s;
    auto matrix = [&](const std::string& n, int64_t r, int64_t k) { s.push_back({n, {r, k}, ParamSpec::Matrix, false, 0.0, 1.0 / std::sqrt(static_cast<double>(k))}); };
    auto vector = [&](const std::string& n, int64_t k, double mean, double std) { s.push_back({n, {k}, ParamSpec::Vector, false, mean, std}); };
    s.push_back({"embed", {c.vocab, D}, ParamSpec::Matrix, false, 0.0, 1.0});
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const MixerConfig& x = l.mix;
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        vector(L + "norm1", D, 1.0, 0.1);
        if (l.mlp.present) vector(L + "norm2", D, 1.0, 0.1);
        if (x.kind == MixerConfig::Attention) {
            matrix(M + "q", x.heads * x.dim, D); vector(M + "q.b", x.heads * x.dim, 0.0, 0.1);
            matrix(M + "k", x.kv_heads * x.dim, D); vector(M + "k.b", x.kv_heads * x.dim, 0.0, 0.1);
            matrix(M + "v", x.kv_heads * x.vdim, D); vector(M + "v.b", x.kv_heads * x.vdim, 0.0, 0.1);
            vector(M + "q.norm", x.heads * x.dim, 1.0, 0.1);
            vector(M + "k.norm", x.kv_heads * x.dim, 1.0, 0.1);
            vector(M + "pb", x.heads, -2.0, 0.5);
            matrix(M + "g", x.heads, D);
            matrix(M + "o", D, x.heads * x.vdim); vector(M + "o.b", D, 0.0, 0.1);
        } else {
            matrix(M + "q", x.heads * x.dim, D);
            matrix(M + "k", x.heads * x.dim, D);
            matrix(M + "v", x.heads * x.vdim, D);
            matrix(M + "g", x.heads * x.vdim, D);
            matrix(M + "o", D, x.heads * x.vdim);
            if (x.kind == MixerConfig::Gla) {
                vector(M + "norm", x.vdim, 1.0, 0.1);
                // (the rank of the decays' map is the checkpoint's to decide: the height of a1, the width of a2)
                s.push_back({M + "a1", {x.rank, D}, ParamSpec::Matrix, false, 0.0, 1.0 / std::sqrt(static_cast<double>(D)), 0.0, 0});
                // (the second half of the map stays fp32: it is applied inside the kernel that makes the decays)
                s.push_back({M + "a2", {x.heads * x.dim, x.rank}, ParamSpec::Vector, false, 0.0, 1.0 / std::sqrt(static_cast<double>(x.rank)), 0.0, 1});
                vector(M + "a2.b", x.heads * x.dim, 2.0, 1.0);
            }
        }
        if (l.mlp.present) {
            const MlpConfig& f = l.mlp;
            for (int64_t e = 0; e < f.experts; ++e) {
                const std::string E = L + "mlp.e" + std::to_string(e) + ".";
                matrix(E + "up", f.ff, D);
                matrix(E + "down", D, f.ff);
            }
            matrix(L + "mlp.router", f.experts, D);
            if (f.shared_ff > 0) {
                matrix(L + "mlp.shared.up", f.shared_ff, D);
                matrix(L + "mlp.shared.down", D, f.shared_ff);
            }
        }
        if (c.taps > 0) {
            s.push_back({L + "canon1", {D, c.taps}, ParamSpec::Vector, false, 0.0, 0.5 / std::sqrt(static_cast<double>(c.taps))});
            if (l.mlp.present) s.push_back({L + "canon2", {D, c.taps}, ParamSpec::Vector, false, 0.0, 0.5 / std::sqrt(static_cast<double>(c.taps))});
        }
        vector(L + "dwa", static_cast<int64_t>(i) + 2, 1.0 / static_cast<double>(i + 2), 0.1);
    }
    vector("final.norm", D, 1.0, 0.1);
    return s;
}

void viladra_assemble(const Json& config, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    ViladraConfig c(config);
    const int D = static_cast<int>(c.width);
    DecoderModel& m = out.model;
    {
        Params e, h;
        e.tensor["table"] = t.at("embed");
        e.num["scale"] = c.embed_scale;
        m.embedding = build_embedding("token_table", e);
        h.tensor["weight"] = t.at("embed");          // the head is the embedding table, without its scale
        h.num["dtype"] = dtype;
        h.num["softcap"] = c.logit_softcap;
        m.head = build_head("linear", h);
    }
    auto norm = [&](const std::string& name) {
        Params p;
        p.num["size"] = D; p.num["eps"] = c.eps; p.num["dtype"] = dtype;
        p.tensor["weight"] = t.at(name);
        return build_norm("rmsnorm", p);
    };
    Tensor2 no_conv;
    Params mix;
    mix.num["passes"] = static_cast<double>(c.layers.size());
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const MixerConfig& x = l.mix;
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        std::unique_ptr<Mixer> mixer;
        Params p;
        p.num["heads"] = static_cast<double>(x.heads); p.num["dim"] = static_cast<double>(x.dim); p.num["value_dim"] = static_cast<double>(x.vdim);
        p.num["eps"] = c.eps; p.num["dtype"] = dtype;
        p.tensor["out.weight"] = t.at(M + "o");
        if (x.kind == MixerConfig::Attention) {
            p.num["kv_heads"] = static_cast<double>(x.kv_heads);
            p.num["scale"] = x.scale; p.num["window"] = static_cast<double>(x.mask);
            p.num["gated"] = 1; p.num["gate_per_head"] = 1; p.num["sigmoid_weights"] = 1;
            p.str["qk_norm"] = "row";
            p.tensor["q.norm"] = t.at(M + "q.norm"); p.tensor["k.norm"] = t.at(M + "k.norm");
            p.tensor["score_bias"] = t.at(M + "pb");
            p.tensor["in.weight"] = out.store.join_rows({t.at(M + "q"), t.at(M + "k"), t.at(M + "v"), t.at(M + "g")});
            // (the gate's projection has no bias)
            auto column = [](const Tensor2& v) { return Tensor2(v.data, v.dtype, v.rows * v.cols, 1); };
            p.tensor["in.bias"] = out.store.join_rows({column(t.at(M + "q.b")), column(t.at(M + "k.b")), column(t.at(M + "v.b")), column(out.store.zeros(x.heads))});
            p.tensor["out.bias"] = t.at(M + "o.b");
            mixer = build_mixer("scored_attention", p);
        } else {
            std::vector<Tensor2> in = {t.at(M + "q"), t.at(M + "k"), t.at(M + "v"), t.at(M + "g")};
            if (x.kind == MixerConfig::Gla) {
                in.push_back(t.at(M + "a1"));
                p.num["q_scale"] = 1.0 / std::sqrt(static_cast<double>(x.dim));
                p.num["tau"] = x.tau;
                p.tensor["decay.weight"] = t.at(M + "a2");
                p.tensor["decay.bias"] = t.at(M + "a2.b");
                p.tensor["norm.weight"] = out.store.repeat(t.at(M + "norm"), static_cast<int>(x.heads));     // one weight, shared by the heads
            } else {
                p.num["k_scale"] = 1.0 / std::sqrt(static_cast<double>(x.dim));
                p.num["rot_dims"] = static_cast<double>(x.rot_dims); p.num["rot_base"] = x.rot_base;
                std::vector<float> decay(x.decay.begin(), x.decay.end());
                p.tensor["head_decay"] = out.store.upload(decay, 1, static_cast<int64_t>(decay.size()), F32);
            }
            p.tensor["in.weight"] = out.store.join_rows(in);
            mixer = build_mixer("linear_attention", p);
        }
        std::unique_ptr<FeedForward> ff;
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(norm(L + "norm1"));
        if (l.mlp.present) {
            const MlpConfig& f = l.mlp;
            Params q;
            q.num["dtype"] = dtype; q.num["experts"] = static_cast<double>(f.experts); q.num["ff"] = static_cast<double>(f.ff);
            q.num["top"] = static_cast<double>(f.top); q.num["scale"] = f.scale;
            q.str["activation"] = "relu2";               // the design fixes the squared ReLU
            std::vector<Tensor2> ups, downs;
            for (int64_t e = 0; e < f.experts; ++e) {
                const std::string E = L + "mlp.e" + std::to_string(e) + ".";
                ups.push_back(t.at(E + "up"));
                downs.push_back(t.at(E + "down"));
            }
            if (f.shared_ff > 0) { ups.push_back(t.at(L + "mlp.shared.up")); downs.push_back(t.at(L + "mlp.shared.down")); }
            q.tensor["up.weight"] = out.store.join_rows(ups);
            q.tensor["down.weight"] = out.store.join_cols(downs);
            q.tensor["router"] = t.at(L + "mlp.router");
            ff = build_feed_forward("routed_experts", q);
            norms.push_back(norm(L + "norm2"));
        }
        Params b;
        b.num["dtype"] = dtype; b.num["size"] = D;
        if (c.taps > 0) {
            b.tensor["mixer_conv"] = t.at(L + "canon1");
            if (l.mlp.present) b.tensor["ff_conv"] = t.at(L + "canon2");
        } else if (dtype != F32) {
            // (no input convolution: one tap of weight zero hands the stream on in the compute dtype)
            if (no_conv.data == nullptr) { const Tensor2 z = out.store.zeros(D); no_conv = Tensor2(z.data, F32, D, 1); }
            b.tensor["mixer_conv"] = no_conv;
            if (l.mlp.present) b.tensor["ff_conv"] = no_conv;
        }
        m.layers.push_back(build_block("post_norm", std::move(mixer), std::move(ff), std::move(norms), b));
        mix.tensor["w" + std::to_string(i)] = t.at(L + "dwa");
    }
    m.stream_steps.push_back(build_stream_step("depth_mix", mix));
    for (int i = 0; i < static_cast<int>(c.layers.size()); ++i) {
        LayerCall lc;
        lc.layer = i; lc.cache = i; lc.write = true; lc.after = 0; lc.after_pass = i;
        m.order.push_back(lc);
    }
    m.final_norm = norm("final.norm");
    out.max_positions = 0;          // positions are not bounded by a table
    if (const Json* e = config.find("eos_token_id")) if (e->is_integer()) out.eos_token_id = static_cast<int>(e->integer());
}

}  // namespace

void register_viladra() {
    Architecture a;
    a.name = "Viladra";
    a.param_specs = viladra_specs;
    a.assemble = viladra_assemble;
    register_architecture(a, "viladra");
}

}  // namespace minillm
