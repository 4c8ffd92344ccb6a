// Piditar: a decoder whose layers are listed one by one in its configuration, each a pre-norm block around one of three
// mixers and an optional dense feed-forward.  "attention": grouped-query attention with biases on q, k and v, rotation by
// neighbouring pairs of a head's first elements, heads divided by their root mean square after the rotation (no weight),
// a score scale of its own and a cap c tanh(s / c), values of their own size.  "rglru": the recurrent block with a
// real-gated linear recurrent unit.  "mamba2": the selective state-space mixer with a scalar decay per head.  A span of
// the layers may run several times in a row with the same weights, every pass with a cache and state of its own and, from
// the second pass on, the embedding's output added to the stream in front of it.  Norms multiply by 1 + w; the embedding
// is scaled and doubles as the head.
//
// This file holds what is particular to the architecture: which config.json keys it reads and how they become a ModelSpec
// with the checkpoint's tensor names.  Nothing here computes.
//
// config.json: architecture "Piditar"; vocab, width; embedding.scale; norm.eps; layers: a list of {type, mixer, mlp};
// loop {start, stop, times} (optional).  mixer of "attention": {heads, kv_heads, dim, vdim, scale, softcap, rot {base, dims}};
// of "rglru": {width, blocks, conv}; of "mamba2": {heads, vdim, state, groups, conv, norm_groups}.  mlp: null or {kind "dense", ff}.
// max_positions (optional): the longest sequence, 131072 unless given.
// Tensors: embed, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mlp.{gate, up, down}; attention: l<i>.mix.{q, k, v, o} and
// {q, k, v}.b; rglru: l<i>.mix.{y, y.b, x, x.b, conv, conv.b, ra, ra.b, ri, ri.b, lam, o}; mamba2: l<i>.mix.{in, conv, conv.b,
// dt_bias, A_log, D, norm, o}.
#include "config.h"

namespace tq {
namespace {

const long long DEFAULT_MAX_POSITIONS = 131072;
const double RGLRU_DECAY_SCALE = 8.0;          // log a = -8 r softplus(lam): fixed by the design

const Json& object_at(const Json& parent, const char* key, const std::string& where) {
    const Json& j = parent[key];
    if (!j.is_object()) raise(TQE_ERR_CONFIG, "%s: '%s' must be an object", where.c_str(), key);
    return j;
}

Json mixer_typed(const Json& raw, const std::string& where, const std::string& type) {
    KeyReader r(raw, where);
    Json m = Json::object();
    if (type == "attention") {
        m.set("heads", r.integer("heads", 1));
        m.set("kv_heads", r.integer("kv_heads", 1));
        m.set("dim", r.integer("dim", 1));
        m.set("vdim", r.integer("vdim", 1));
        m.set("scale", r.number("scale", true));
        m.set("softcap", r.has("softcap") ? Json(r.number("softcap", true)) : Json());
        if (m["heads"].as_int() % m["kv_heads"].as_int())
            raise(TQE_ERR_CONFIG, "%s: %lld heads are not a multiple of %lld kv_heads", where.c_str(), (long long)m["heads"].as_int(), (long long)m["kv_heads"].as_int());
        KeyReader rot(object_at(raw, "rot", where), where + ".rot");
        const long long dims = rot.integer("dims", 0);
        if (dims % 2 || dims > m["dim"].as_int()) raise(TQE_ERR_CONFIG, "%s.rot: dims %lld must be even and at most dim %lld", where.c_str(), dims, (long long)m["dim"].as_int());
        m.set("rot_base", rot.number("base", true));
        m.set("rot_dims", dims);
    } else if (type == "rglru") {
        m.set("width", r.integer("width", 1));
        m.set("blocks", r.integer("blocks", 1));
        m.set("conv", r.integer("conv", 1));
        if (m["width"].as_int() % m["blocks"].as_int())
            raise(TQE_ERR_CONFIG, "%s: a width of %lld does not fall into %lld blocks", where.c_str(), (long long)m["width"].as_int(), (long long)m["blocks"].as_int());
    } else {
        m.set("heads", r.integer("heads", 1));
        m.set("vdim", r.integer("vdim", 1));
        m.set("state", r.integer("state", 1));
        m.set("groups", r.integer("groups", 1));
        m.set("conv", r.integer("conv", 1));
        m.set("norm_groups", r.integer("norm_groups", 1));
        if (m["heads"].as_int() % m["groups"].as_int())
            raise(TQE_ERR_CONFIG, "%s: %lld heads do not fall into %lld groups", where.c_str(), (long long)m["heads"].as_int(), (long long)m["groups"].as_int());
        if ((m["heads"].as_int() * m["vdim"].as_int()) % m["norm_groups"].as_int())
            raise(TQE_ERR_CONFIG, "%s: heads x vdim does not fall into %lld norm_groups", where.c_str(), (long long)m["norm_groups"].as_int());
    }
    return m;
}

Json mlp_typed(const Json& raw, const std::string& where) {
    if (raw.is_null()) return Json();
    if (!raw.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object or null", where.c_str());
    KeyReader r(raw, where);
    const std::string kind = r.string("kind");
    if (kind != "dense") raise(TQE_ERR_CONFIG, "%s: unknown kind '%s' (known: dense)", where.c_str(), kind.c_str());
    Json m = Json::object();
    m.set("kind", kind);
    m.set("ff", r.integer("ff", 1));
    return m;
}

Json piditar_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    Json c = Json::object();
    c.set("vocab", r.integer("vocab", 1));
    c.set("width", r.integer("width", 1));
    c.set("embedding_scale", KeyReader(object_at(raw, "embedding", where), where + ": embedding").number("scale"));
    c.set("norm_eps", KeyReader(object_at(raw, "norm", where), where + ": norm").number("eps"));
    c.set("max_positions", r.integer_or("max_positions", DEFAULT_MAX_POSITIONS, 1));
    if (!raw["layers"].is_array() || raw["layers"].items().empty()) raise(TQE_ERR_CONFIG, "%s: 'layers' must be a list of at least one layer", where.c_str());
    Json list = Json::array();
    long long i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string at = format("%s: layers[%lld]", where.c_str(), i++);
        if (!l.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object", at.c_str());
        const std::string type = KeyReader(l, at).string("type");
        if (type != "attention" && type != "rglru" && type != "mamba2")
            raise(TQE_ERR_CONFIG, "%s: unknown type '%s' (known: attention, mamba2, rglru)", at.c_str(), type.c_str());
        Json t = Json::object();
        t.set("type", type);
        t.set("mixer", mixer_typed(object_at(l, "mixer", at), at + ".mixer", type));
        t.set("mlp", mlp_typed(l["mlp"], at + ".mlp"));
        list.push(t);
    }
    c.set("layers", list);
    // the span of layers that runs several times; absent: every layer once
    long long start = 0, stop = 0, times = 1;
    if (!raw["loop"].is_null()) {
        KeyReader loop(object_at(raw, "loop", where), where + ": loop");
        start = loop.integer("start", 0);
        stop = loop.integer("stop", 0);
        times = loop.integer("times", 1);
        if (start > stop || stop > i) raise(TQE_ERR_CONFIG, "%s: loop: layers %lld to %lld of %lld", where.c_str(), start, stop, i);
        if (times * (stop - start) > 100000) raise(TQE_ERR_CONFIG, "%s: loop: %lld passes over %lld layers are too many", where.c_str(), times, stop - start);
    }
    c.set("loop_start", start);
    c.set("loop_stop", stop);
    c.set("loop_times", times);
    return c;
}

PartSpec part(const char* kind, std::initializer_list<std::pair<const char*, Json>> params) {
    PartSpec p;
    p.kind = kind;
    for (const auto& kv : params) p.params.set(kv.first, kv.second);
    return p;
}

Json names_of(std::initializer_list<std::pair<const char*, const char*>> pairs) {
    Json n = Json::object();
    for (const auto& kv : pairs) n.set(kv.first, kv.second);
    return n;
}

ModelSpec piditar_spec(const Json& c) {
    const long long width = c["width"].as_int();
    const PartSpec norm = part("rms_norm", {{"size", width}, {"eps", c["norm_eps"]}, {"unit_offset", true}, {"tensor", ""}});
    ModelSpec s;
    s.architecture = "Piditar";
    s.vocab_size = c["vocab"].as_int();
    s.hidden_size = width;
    s.max_positions = c["max_positions"].as_int();
    s.embedding_name = "embed";
    s.has_embedding_scale = true;
    s.embedding_scale = c["embedding_scale"].as_number();
    size_t l = 0;
    for (const Json& layer : c["layers"].items()) {
        const Json& m = layer["mixer"];
        const Json& mlp = layer["mlp"];
        const std::string type = layer["type"].as_string();
        PartSpec mixer;
        if (type == "attention") {
            const PartSpec position = m["rot_dims"].as_int() > 0
                ? part("rotary", {{"theta", m["rot_base"]}, {"rot_dim", m["rot_dims"]}, {"max_positions", c["max_positions"]}, {"style", "pairs"}})
                : part("none", {{"max_positions", c["max_positions"]}});
            mixer = part("attention", {{"hidden", width}, {"n_heads", m["heads"]}, {"n_kv_heads", m["kv_heads"]}, {"head_dim", m["dim"]}, {"value_dim", m["vdim"]},
                                       {"scale", m["scale"]}, {"qkv_bias", true}, {"qk_norm", true}, {"qk_norm_weight", false}, {"qk_norm_after_rotation", true},
                                       {"eps", c["norm_eps"]}, {"cap", m["softcap"]}, {"position", position.to_json()},
                                       {"names", names_of({{"q", "q"}, {"k", "k"}, {"v", "v"}, {"o", "o"}, {"q_bias", "q.b"}, {"k_bias", "k.b"}, {"v_bias", "v.b"}})}});
        } else if (type == "rglru") {
            mixer = part("rglru", {{"hidden", width}, {"width", m["width"]}, {"blocks", m["blocks"]}, {"conv", m["conv"]}, {"decay_scale", RGLRU_DECAY_SCALE},
                                   {"names", names_of({{"y", "y"}, {"y_bias", "y.b"}, {"x", "x"}, {"x_bias", "x.b"}, {"conv", "conv"}, {"conv_bias", "conv.b"},
                                                       {"gate_a", "ra"}, {"gate_a_bias", "ra.b"}, {"gate_i", "ri"}, {"gate_i_bias", "ri.b"}, {"decay", "lam"}, {"o", "o"}})}});
        } else {
            mixer = part("mamba2", {{"hidden", width}, {"heads", m["heads"]}, {"head_dim", m["vdim"]}, {"state", m["state"]}, {"groups", m["groups"]},
                                    {"conv", m["conv"]}, {"norm_groups", m["norm_groups"]}, {"eps", c["norm_eps"]},
                                    {"names", names_of({{"in", "in"}, {"conv", "conv"}, {"conv_bias", "conv.b"}, {"dt_bias", "dt_bias"}, {"a_log", "A_log"}, {"d", "D"},
                                                        {"norm", "norm"}, {"o", "o"}})}});
        }
        Json ff;
        if (!mlp.is_null())
            ff = part("gated", {{"hidden", width}, {"inter", mlp["ff"]}, {"gate", "silu"}, {"names", names_of({{"gate", "gate"}, {"up", "up"}, {"down", "down"}})}}).to_json();
        LayerSpec spec;
        spec.prefix = format("l%zu.", l++);
        spec.block = part("pre_norm", {{"mixer", mixer.to_json()}, {"feed_forward", ff}, {"mixer_norm", norm.to_json()}, {"ff_norm", mlp.is_null() ? Json() : norm.to_json()},
                                       {"names", names_of({{"mixer", "mix."}, {"feed_forward", "mlp."}, {"mixer_norm", "norm1"}, {"ff_norm", "norm2"}})}});
        s.layers.push_back(spec);
    }
    // the run order: the layers before the span, the span `times` times, the rest
    const long long n = (long long)s.layers.size(), start = c["loop_start"].as_int(), stop = c["loop_stop"].as_int(), times = c["loop_times"].as_int();
    auto run_of = [](long long layer, bool add) { Run r; r.layer = (int)layer; r.add_embedding = add; return r; };
    for (long long i = 0; i < start; ++i) s.order.push_back(run_of(i, false));
    for (long long pass = 0; pass < times; ++pass)
        for (long long i = start; i < stop; ++i) s.order.push_back(run_of(i, pass > 0 && i == start));
    for (long long i = stop; i < n; ++i) s.order.push_back(run_of(i, false));
    s.final_norm = norm;
    s.final_norm_prefix = "final.norm";
    s.head_name = "";
    return s;
}

}  // namespace

void register_piditar() {
    Architecture a;
    a.name = "Piditar";
    a.model_types = {"piditar"};
    a.typed_config = piditar_typed;
    a.build_spec = piditar_spec;
    register_architecture(a);
}

}  // namespace tq
