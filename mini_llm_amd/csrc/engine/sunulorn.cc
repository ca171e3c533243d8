// Sunulorn: a decoder whose configuration lists its layers one by one. A layer adds a mixer's and a feed-forward's
// result to the residual stream, both computed from the same stream, each behind an RMS norm of its own. The mixer is
// one of three softmax attentions with grouped heads: "attention" (a short causal convolution over the projected
// queries and keys, the keys behind it are the values too, interleaved rotary pairs, one more term exp(0) in the
// softmax's denominator), "attention_2" (biases, half-split rotary pairs, queries and keys at unit root mean square
// per head behind the rotation, a sliding window that also keeps the sequence's first positions, a gate per output
// column) and "attention_3" (biases, a distance penalty whose slope the head's index fixes, a learned sink per head in
// the denominator, a gate per head, optionally the keys and values of an earlier layer). The feed-forward is gated
// (silu), or a mixture of clamped gated experts chosen by sigmoid scores that multiply the expert's input, beside a
// shared expert scaled by a sigmoid of the input. The embedding is scaled; the head is a matrix of its own behind a
// final norm. This file reads the configuration, names the tensors and chooses the parts; the mechanisms are the
// parts' own.
//
// config.json: {"architecture": "Sunulorn", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"},
//   "layers": [{"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv", "rot": {"base", "dims"}, "scale"}, "mlp": ...},
//              {"type": "attention_2", "mixer": {"heads", "kv_heads", "dim", "vdim", "rot": {..}, "scale", "mask": {"size", "keep_first"}}, "mlp": ...},
//              {"type": "attention_3", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", ["kv_from": j]}, "mlp": ...}]}
//   mlp: {"kind": "dense", "ff"} | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff", "limit"},
//         "shared": {"ff", "limit"} | null} | null
//   May be absent: embedding (scale 1), kv_heads (as many as heads), vdim (as wide as dim), conv (none), rot (none),
//   mask (plain causal), mask.keep_first (0), kv_from, mlp.kind (dense), mlp.shared, mlp.
// Tensors: embed, head, final.norm, l<i>.norm1[/norm2], l<i>.mix.{q, k, v, g, o}[.b], l<i>.mix.{q,k}.conv, l<i>.mix.sink,
// l<i>.mlp.{gate, up, down} or l<i>.mlp.{router, e<k>.{gate, up, down}, shared.{gate, up, down, sg}}; linear weights are
// stored [out, in].
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
// an optional object: null and absent are the same
const Json* optional_object(const Json& c, const char* key, const std::string& where) {
    const Json* v = c.find(key);
    if (v == nullptr || v->is_null()) return nullptr;
    if (!v->is_object()) throw ConfigError("config.json: " + where + "'" + key + "' must be an object or null");
    return v;
}

struct MixerConfig {
    enum Kind { ConvAttention, WindowAttention, SinkAttention } kind = ConvAttention;
    int64_t heads = 0, kv_heads = 0, dim = 0, vdim = 0, taps = 0, rot_dims = 0, window = 0, keep_first = 0, kv_from = -1;
    double scale = 1.0, rot_base = 10000.0;
};
struct MlpConfig {
    enum Kind { None, Dense, Moe } kind = None;
    int64_t ff = 0, experts = 0, top = 0, shared_ff = 0;      // shared_ff 0: no shared expert
    double limit = 0.0, shared_limit = 0.0;
};
struct LayerConfig {
    MixerConfig mix;
    MlpConfig mlp;
};

// The constants the design fixes.
const double kGateSlope = 1.702;                  // an expert's gate: g sigmoid(1.702 g)
double head_slope(int64_t h, int64_t heads) {     // the distance penalty of head h of `heads`
    return std::exp2(-8.0 * static_cast<double>(h + 1) / static_cast<double>(heads));
}

struct SunulornConfig {
    int64_t vocab = 0, width = 0;
    double eps = 1e-6, embed_scale = 1.0;
    std::vector<LayerConfig> layers;

    explicit SunulornConfig(const Json& c) {
        vocab = need_int(c, "vocab", "");
        width = need_int(c, "width", "");
        eps = need_num(need_object(c, "norm", ""), "eps", "norm: ");
        if (!(eps > 0)) throw ConfigError("config.json: norm.eps must be positive");
        if (const Json* e = optional_object(c, "embedding", "")) embed_scale = need_num(*e, "scale", "embedding: ");
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
            x.heads = need_int(m, "heads", where);
            x.kv_heads = m.find("kv_heads") != nullptr ? need_int(m, "kv_heads", where) : x.heads;
            if (x.heads % x.kv_heads != 0) throw ConfigError("config.json: " + where + "heads is not a multiple of kv_heads");
            x.dim = need_int(m, "dim", where);
            x.vdim = m.find("vdim") != nullptr ? need_int(m, "vdim", where) : x.dim;
            x.scale = need_num(m, "scale", where);
            auto rotation = [&]() {
                if (const Json* rot = optional_object(m, "rot", where)) {
                    x.rot_base = need_num(*rot, "base", where + "rot: ");
                    x.rot_dims = need_int(*rot, "dims", where + "rot: ", 0);
                    if (!(x.rot_base > 0) || x.rot_dims % 2 != 0 || x.rot_dims > x.dim)
                        throw ConfigError("config.json: " + where + "rot.base must be positive, rot.dims even and at most dim");
                }
            };
            if (type->string() == "attention") {
                x.kind = MixerConfig::ConvAttention;
                if (x.vdim != x.dim) throw ConfigError("config.json: " + where + "the values are the keys: vdim must equal dim");
                if (const Json* taps = m.find("conv")) {
                    if (!taps->is_null()) {
                        x.taps = need_int(m, "conv", where, 0);           // (0: none, as when the key is absent)
                        if (x.taps > 16) throw ConfigError("config.json: " + where + "a convolution of more than 16 taps is not supported");
                    }
                }
                rotation();
            } else if (type->string() == "attention_2") {
                x.kind = MixerConfig::WindowAttention;
                rotation();
                if (const Json* mask = optional_object(m, "mask", where)) {
                    x.window = need_int(*mask, "size", where + "mask: ");
                    if (mask->find("keep_first") != nullptr && !mask->find("keep_first")->is_null()) x.keep_first = need_int(*mask, "keep_first", where + "mask: ", 0);
                }
            } else if (type->string() == "attention_3") {
                x.kind = MixerConfig::SinkAttention;
                if (const Json* from = m.find("kv_from")) {
                    if (!from->is_null()) {
                        if (!from->is_integer() || from->integer() < 0 || from->integer() >= static_cast<int64_t>(i))
                            throw ConfigError("config.json: " + where + "kv_from must name an earlier layer");
                        x.kv_from = from->integer();
                        const MixerConfig& src = layers[static_cast<size_t>(x.kv_from)].mix;
                        if (src.kind != MixerConfig::SinkAttention || src.kv_from >= 0)
                            throw ConfigError("config.json: " + where + "kv_from must name an attention_3 layer with keys and values of its own");
                        if (src.kv_heads != x.kv_heads || src.dim != x.dim || src.vdim != x.vdim)
                            throw ConfigError("config.json: " + where + "kv_heads, dim and vdim must equal those of the layer kv_from names");
                    }
                }
            } else {
                throw ConfigError("config.json: " + where + "unknown layer type '" + type->string() + "' (known: attention, attention_2, attention_3)");
            }
            if (const Json* mlp = optional_object(l, "mlp", where)) {
                MlpConfig& f = lc.mlp;
                std::string kind = "dense";
                if (const Json* k = mlp->find("kind")) {
                    if (!k->is_string()) throw ConfigError("config.json: " + where + "mlp.kind must be a string");
                    kind = k->string();
                }
                if (kind == "dense") {
                    f.kind = MlpConfig::Dense;
                    f.ff = need_int(*mlp, "ff", where + "mlp: ");
                } else if (kind == "moe") {
                    f.kind = MlpConfig::Moe;
                    const Json& r = need_object(*mlp, "router", where + "mlp: ");
                    f.experts = need_int(r, "experts", where + "mlp: router: ");
                    f.top = need_int(r, "top", where + "mlp: router: ");
                    if (f.top > f.experts) throw ConfigError("config.json: " + where + "mlp: router.top exceeds router.experts");
                    if (f.experts > 256) throw ConfigError("config.json: " + where + "mlp: more than 256 experts are not supported");
                    const Json& e = need_object(*mlp, "expert", where + "mlp: ");
                    f.ff = need_int(e, "ff", where + "mlp: expert: ");
                    f.limit = need_num(e, "limit", where + "mlp: expert: ");
                    if (!(f.limit > 0)) throw ConfigError("config.json: " + where + "mlp: expert.limit must be positive");
                    if (const Json* sh = optional_object(*mlp, "shared", where + "mlp: ")) {
                        f.shared_ff = need_int(*sh, "ff", where + "mlp: shared: ");
                        f.shared_limit = need_num(*sh, "limit", where + "mlp: shared: ");
                        if (!(f.shared_limit > 0)) throw ConfigError("config.json: " + where + "mlp: shared.limit must be positive");
                    }
                } else {
                    throw ConfigError("config.json: " + where + "mlp.kind must be 'dense' or 'moe'");
                }
            }
            layers.push_back(lc);
        }
    }
};

std::vector<ParamSpec> sunulorn_specs(const Json& config) {
    const SunulornConfig c(config);
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
        if (l.mlp.kind != MlpConfig::None) vector(L + "norm2", D, 1.0, 0.1);
        const bool biases = x.kind != MixerConfig::ConvAttention;
        matrix(M + "q", x.heads * x.dim, D);
        if (biases) vector(M + "q.b", x.heads * x.dim, 0.0, 0.1);
        if (x.kv_from < 0) {
            matrix(M + "k", x.kv_heads * x.dim, D);
            if (biases) vector(M + "k.b", x.kv_heads * x.dim, 0.0, 0.1);
            if (x.kind != MixerConfig::ConvAttention) {
                matrix(M + "v", x.kv_heads * x.vdim, D);
                vector(M + "v.b", x.kv_heads * x.vdim, 0.0, 0.1);
            }
        }
        if (x.kind == MixerConfig::ConvAttention && x.taps > 0) {
            s.push_back({M + "q.conv", {x.heads * x.dim, x.taps}, ParamSpec::Vector, false, 0.0, 1.0 / std::sqrt(static_cast<double>(x.taps))});
            s.push_back({M + "k.conv", {x.kv_heads * x.dim, x.taps}, ParamSpec::Vector, false, 0.0, 1.0 / std::sqrt(static_cast<double>(x.taps))});
        }
        if (x.kind == MixerConfig::WindowAttention) matrix(M + "g", x.heads * x.vdim, D);
        if (x.kind == MixerConfig::SinkAttention) {
            vector(M + "sink", x.heads, 0.0, 1.0);
            matrix(M + "g", x.heads, D);
        }
        matrix(M + "o", D, x.heads * x.vdim);
        if (x.kind == MixerConfig::WindowAttention) vector(M + "o.b", D, 0.0, 0.1);
        const MlpConfig& f = l.mlp;
        auto expert = [&](const std::string& E, int64_t ff) {
            matrix(E + "gate", ff, D);
            matrix(E + "up", ff, D);
            matrix(E + "down", D, ff);
        };
        if (f.kind == MlpConfig::Dense) expert(L + "mlp.", f.ff);
        if (f.kind == MlpConfig::Moe) {
            for (int64_t e = 0; e < f.experts; ++e) expert(L + "mlp.e" + std::to_string(e) + ".", f.ff);
            matrix(L + "mlp.router", f.experts, D);
            if (f.shared_ff > 0) {
                expert(L + "mlp.shared.", f.shared_ff);
                matrix(L + "mlp.shared.sg", 1, D);
            }
        }
    }
    vector("final.norm", D, 1.0, 0.1);
    matrix("head", c.vocab, D);
    return s;
}

void sunulorn_assemble(const Json& config, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const SunulornConfig c(config);
    const int D = static_cast<int>(c.width);
    DecoderModel& m = out.model;
    {
        Params e, h;
        e.tensor["table"] = t.at("embed");
        e.num["scale"] = c.embed_scale;
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
    auto column = [](const Tensor2& v) { return Tensor2(v.data, v.dtype, v.rows * v.cols, 1); };
    for (size_t i = 0; i < c.layers.size(); ++i) {
        const LayerConfig& l = c.layers[i];
        const MixerConfig& x = l.mix;
        const std::string L = "l" + std::to_string(i) + ".", M = L + "mix.";
        // Value heads narrower than the keys are made as wide: zero rows in the values' projection (and the gate's), zero
        // columns in the output projection. The result is the same, and the attention kernels that every model shares
        // (key tiles on the matrix cores, split keys) take keys and values of one width only.
        // Value heads WIDER than the keys: the queries' and keys' heads get zero columns instead (zero rows in their
        // projections and biases); the dot products are the same. Where queries and keys are scaled to unit root mean
        // square over the head, the wider head's mean is dim / d times the true one, so eps * dim / d stands for eps
        // and the normed vectors come out sqrt(d / dim) times too long, which scale * dim / d takes back:
        //   x / sqrt(sum / d + eps dim / d) = sqrt(d / dim) x / sqrt(sum / dim + eps).
        const int64_t e = (x.vdim < x.dim && x.dim % 16 == 0) ? x.dim : x.vdim;
        const int64_t d = (x.vdim > x.dim && x.vdim % 16 == 0 && x.kind != MixerConfig::ConvAttention) ? x.vdim : x.dim;
        auto widened_rows = [&](const Tensor2& w) { return e == x.vdim ? w : out.store.pad_row_blocks(w, x.vdim, e); };
        auto widened_keys = [&](const Tensor2& w) { return d == x.dim ? w : out.store.pad_row_blocks(w, x.dim, d); };
        const double shrink = static_cast<double>(x.dim) / static_cast<double>(d);
        const bool unit_norm = x.kind == MixerConfig::WindowAttention;
        Params p;
        p.num["heads"] = static_cast<double>(x.heads); p.num["kv_heads"] = static_cast<double>(x.kv_heads);
        p.num["dim"] = static_cast<double>(d); p.num["value_dim"] = static_cast<double>(e);
        p.num["scale"] = unit_norm ? x.scale * shrink : x.scale; p.num["eps"] = unit_norm ? c.eps * shrink : c.eps; p.num["dtype"] = dtype;
        p.str["qk_norm"] = "none";
        p.tensor["out.weight"] = e == x.vdim ? t.at(M + "o") : out.store.pad_col_blocks(t.at(M + "o"), x.vdim, e);
        if (x.kind == MixerConfig::ConvAttention) {
            p.num["values_from_keys"] = 1;
            p.num["rot_dims"] = static_cast<double>(x.rot_dims); p.num["rot_base"] = x.rot_base; p.num["rot_interleaved"] = 1;
            p.tensor["sink"] = out.store.zeros(x.heads);          // the denominator's extra term is exp(0)
            p.tensor["in.weight"] = out.store.join_rows({t.at(M + "q"), t.at(M + "k")});
            // (a convolution of one tap is a scale per channel; it needs no state but is applied all the same)
            if (x.taps > 0) p.tensor["qk_conv"] = out.store.join_rows({t.at(M + "q.conv"), t.at(M + "k.conv")});
        } else if (x.kind == MixerConfig::WindowAttention) {
            p.num["rot_dims"] = static_cast<double>(x.rot_dims); p.num["rot_base"] = x.rot_base;
            p.str["qk_norm"] = "unit_after";
            p.num["window"] = static_cast<double>(x.window); p.num["keep_first"] = static_cast<double>(x.window > 0 ? x.keep_first : 0);
            p.num["gated"] = 1;
            p.tensor["in.weight"] = out.store.join_rows({widened_keys(t.at(M + "q")), widened_keys(t.at(M + "k")), widened_rows(t.at(M + "v")), widened_rows(t.at(M + "g"))});
            // (the gate's projection has no bias)
            p.tensor["in.bias"] = out.store.join_rows({widened_keys(column(t.at(M + "q.b"))), widened_keys(column(t.at(M + "k.b"))), widened_rows(column(t.at(M + "v.b"))), column(out.store.zeros(x.heads * e))});
            p.tensor["out.bias"] = t.at(M + "o.b");
        } else {
            p.num["gated"] = 1; p.num["gate_per_head"] = 1;
            p.tensor["sink"] = t.at(M + "sink");
            std::vector<float> slopes;
            for (int64_t h = 0; h < x.heads; ++h) slopes.push_back(static_cast<float>(head_slope(h, x.heads)));
            p.tensor["distance_slope"] = out.store.upload(slopes, 1, static_cast<int64_t>(slopes.size()), F32);
            if (x.kv_from >= 0) {
                p.num["shared_kv"] = 1;
                p.tensor["in.weight"] = out.store.join_rows({widened_keys(t.at(M + "q")), t.at(M + "g")});
                p.tensor["in.bias"] = out.store.join_rows({widened_keys(column(t.at(M + "q.b"))), column(out.store.zeros(x.heads))});
            } else {
                p.tensor["in.weight"] = out.store.join_rows({widened_keys(t.at(M + "q")), widened_keys(t.at(M + "k")), widened_rows(t.at(M + "v")), t.at(M + "g")});
                p.tensor["in.bias"] = out.store.join_rows({widened_keys(column(t.at(M + "q.b"))), widened_keys(column(t.at(M + "k.b"))), widened_rows(column(t.at(M + "v.b"))), column(out.store.zeros(x.heads))});
            }
        }
        std::unique_ptr<Mixer> mixer = build_mixer("scored_attention", p);
        std::unique_ptr<FeedForward> ff;
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(norm(L + "norm1"));
        const MlpConfig& f = l.mlp;
        if (f.kind == MlpConfig::Dense) {
            Params q;
            q.num["dtype"] = dtype;
            q.str["activation"] = "silu";
            q.tensor["gate_up.weight"] = out.store.join_rows({t.at(L + "mlp.gate"), t.at(L + "mlp.up")});
            q.tensor["down.weight"] = t.at(L + "mlp.down");
            ff = build_feed_forward("gated_mlp", q);
        } else if (f.kind == MlpConfig::Moe) {
            Params q;
            q.num["dtype"] = dtype; q.num["experts"] = static_cast<double>(f.experts); q.num["ff"] = static_cast<double>(f.ff);
            q.num["top"] = static_cast<double>(f.top);
            q.str["activation"] = "clamped_glu"; q.str["router"] = "sigmoid";
            q.num["limit"] = f.limit; q.num["alpha"] = kGateSlope; q.num["weight_on_input"] = 1;
            std::vector<Tensor2> ups, downs, router = {t.at(L + "mlp.router")};
            for (int64_t e = 0; e < f.experts; ++e) {
                const std::string E = L + "mlp.e" + std::to_string(e) + ".";
                ups.push_back(t.at(E + "gate")); ups.push_back(t.at(E + "up"));
                downs.push_back(t.at(E + "down"));
            }
            if (f.shared_ff > 0) {
                ups.push_back(t.at(L + "mlp.shared.gate")); ups.push_back(t.at(L + "mlp.shared.up"));
                downs.push_back(t.at(L + "mlp.shared.down"));
                router.push_back(t.at(L + "mlp.shared.sg"));          // the shared expert's gate is one more row of the router's product
                q.num["shared_limit"] = f.shared_limit; q.num["shared_gate"] = 1;
            }
            q.tensor["up.weight"] = out.store.join_rows(ups);
            q.tensor["down.weight"] = out.store.join_cols(downs);
            q.tensor["router"] = out.store.join_rows(router);
            ff = build_feed_forward("routed_experts", q);
        }
        if (ff) norms.push_back(norm(L + "norm2"));
        m.layers.push_back(build_block("parallel_norm", std::move(mixer), std::move(ff), std::move(norms)));
    }
    // a layer that takes another's keys and values reads that layer's cache and writes none
    for (int i = 0; i < static_cast<int>(c.layers.size()); ++i) {
        const int64_t from = c.layers[static_cast<size_t>(i)].mix.kv_from;
        LayerCall lc;
        lc.layer = i; lc.cache = from >= 0 ? static_cast<int>(from) : i; lc.write = from < 0;
        m.order.push_back(lc);
    }
    m.final_norm = norm("final.norm");
    out.max_positions = 0;          // positions are not bounded by a table
    if (const Json* e = config.find("eos_token_id")) if (e->is_integer()) out.eos_token_id = static_cast<int>(e->integer());
}

}  // namespace

void register_sunulorn() {
    Architecture a;
    a.name = "Sunulorn";
    a.param_specs = sunulorn_specs;
    a.assemble = sunulorn_assemble;
    register_architecture(a, "sunulorn");
}

}  // namespace minillm
