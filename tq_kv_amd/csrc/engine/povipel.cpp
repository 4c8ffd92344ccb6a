// Povipel: a decoder whose layers are listed one by one in its configuration.  The residual stream is kept in `streams` copies that every
// sublayer reads as a weighted sum and updates all at once (a plain residual sum where the configuration names no streams); a sublayer
// is a layer norm (weight and bias), then the part; what a mixer reads is first mixed with the previous token's, channel by channel.
// Two mixers.  "parallel": two mixers side by side whose outputs are normed over the width, added and halved: a grouped-query
// attention over a sliding window plus one pooled key and value per block of positions in front of the window, with normed heads,
// rotation by neighbouring pairs, values turned by their position and turned back on the way out, and a sink; and a gated linear
// attention whose state decays per key channel by sigmoid(low-rank product)^(1/tau).  "retention": linear attention with a fixed decay
// per head, q and k turned in halves, heads normed without a weight.  Feed-forwards: dense (down gelu_tanh(up)), or routed experts
// scored by a sigmoid each, the weight on the expert's input; or absent.  A span of layers may run several times in a row with the same
// weights, every pass with a cache and state of its own.  The logits are capped, c tanh(l / c).
//
// This file holds what is particular to the architecture: which config.json keys it reads and how they become a ModelSpec with the
// checkpoint's tensor names.  Nothing here computes.
//
// config.json: architecture "Povipel"; vocab, width; embedding.scale; norm.eps; streams (optional); logit_softcap (optional); layers:
// a list of {type, mixer, mlp}; loop {start, stop, times} (optional).  mixer of "parallel": {left {heads, kv_heads, dim, vdim, scale,
// mask {size, pool}, rot {base, dims}}, right {heads, dim, vdim, tau}}; of "retention": {heads, dim, vdim, decay (a list), rot {base,
// dims}}.  mlp: null, {kind "dense", ff} or {kind "moe", expert {ff}, router {experts, top}}.  max_positions (optional): the longest
// sequence, 131072 unless given.
// Tensors: embed, head, final.norm (+ .b), l<i>.norm1, l<i>.norm2 (+ .b), l<i>.shift, l<i>.hc1.{in, out, mix}, l<i>.hc2.{in, out, mix};
// parallel: l<i>.mix.left.{q, k, v, o, q.norm, k.norm, sink}, l<i>.mix.right.{q, k, v, g, o, norm, a1, a2, a2.b}, l<i>.mix.left.out,
// l<i>.mix.right.out; retention: l<i>.mix.{q, k, v, g, o}; dense: l<i>.mlp.{up, down}; moe: l<i>.mlp.router, l<i>.mlp.e<j>.{gate, up, down}.
#include <math.h>

#include "config.h"

namespace tq {
namespace {

const long long DEFAULT_MAX_POSITIONS = 131072;
const long long DEFAULT_DECAY_RANK = 16;        // what random weights get: the checkpoint's tensors give the rank
const double PARALLEL_SCALE = 0.5;              // half the sum of the two mixers: fixed by the design

const Json& object_at(const Json& parent, const char* key, const std::string& where) {
    const Json& j = parent[key];
    if (!j.is_object()) raise(TQE_ERR_CONFIG, "%s: '%s' must be an object", where.c_str(), key);
    return j;
}

void rot_typed(const Json& raw, const std::string& where, long long dim, Json& m) {
    KeyReader rot(object_at(raw, "rot", where), where + ".rot");
    const long long dims = rot.integer("dims", 0);
    if (dims % 2 || dims > dim) raise(TQE_ERR_CONFIG, "%s.rot: dims %lld must be even and at most dim %lld", where.c_str(), dims, dim);
    m.set("rot_base", rot.number("base", true));
    m.set("rot_dims", dims);
}

Json mixer_typed(const Json& raw, const std::string& where, const std::string& type) {
    Json m = Json::object();
    if (type == "parallel") {
        const std::string lw = where + ".left", rw = where + ".right";
        KeyReader l(object_at(raw, "left", where), lw);
        Json left = Json::object();
        left.set("heads", l.integer("heads", 1));
        left.set("kv_heads", l.integer("kv_heads", 1));
        left.set("dim", l.integer("dim", 1));
        left.set("vdim", l.integer("vdim", 1));
        left.set("scale", l.number("scale", true));
        if (left["heads"].as_int() % left["kv_heads"].as_int())
            raise(TQE_ERR_CONFIG, "%s: %lld heads are not a multiple of %lld kv_heads", lw.c_str(), (long long)left["heads"].as_int(), (long long)left["kv_heads"].as_int());
        if (left["vdim"].as_int() % 2) raise(TQE_ERR_CONFIG, "%s: values of %lld elements cannot be turned pair by pair", lw.c_str(), (long long)left["vdim"].as_int());
        KeyReader mask(object_at(l.raw(), "mask", lw), lw + ".mask");
        left.set("window", mask.integer("size", 1));
        left.set("pool", mask.integer("pool", 1));
        rot_typed(l.raw(), lw, left["dim"].as_int(), left);
        KeyReader r(object_at(raw, "right", where), rw);
        Json right = Json::object();
        right.set("heads", r.integer("heads", 1));
        right.set("dim", r.integer("dim", 1));
        right.set("vdim", r.integer("vdim", 1));
        right.set("tau", r.number("tau", true));
        m.set("left", left);
        m.set("right", right);
    } else {
        KeyReader r(raw, where);
        m.set("heads", r.integer("heads", 1));
        m.set("dim", r.integer("dim", 1));
        m.set("vdim", r.integer("vdim", 1));
        const Json& decay = raw["decay"];
        if (!decay.is_array() || (long long)decay.items().size() != m["heads"].as_int())
            raise(TQE_ERR_CONFIG, "%s: 'decay' must list one number for each of the %lld heads", where.c_str(), (long long)m["heads"].as_int());
        Json list = Json::array();
        for (const Json& v : decay.items()) {
            if (!v.is_number()) raise(TQE_ERR_CONFIG, "%s: 'decay' holds something that is no number", where.c_str());
            list.push(Json(v.as_number()));
        }
        m.set("decay", list);
        rot_typed(raw, where, m["dim"].as_int(), m);
    }
    return m;
}

Json mlp_typed(const Json& raw, const std::string& where) {
    if (raw.is_null()) return Json();
    if (!raw.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object or null", where.c_str());
    KeyReader r(raw, where);
    const std::string kind = r.string("kind");
    Json m = Json::object();
    m.set("kind", kind);
    if (kind == "dense") {
        m.set("ff", r.integer("ff", 1));
    } else if (kind == "moe") {
        m.set("ff", KeyReader(object_at(raw, "expert", where), where + ".expert").integer("ff", 1));
        KeyReader router(object_at(raw, "router", where), where + ".router");
        m.set("experts", router.integer("experts", 1));
        m.set("top", router.integer("top", 1));
        if (m["top"].as_int() > m["experts"].as_int())
            raise(TQE_ERR_CONFIG, "%s.router: top %lld of %lld experts", where.c_str(), (long long)m["top"].as_int(), (long long)m["experts"].as_int());
    } else {
        raise(TQE_ERR_CONFIG, "%s: unknown kind '%s' (known: dense, moe)", where.c_str(), kind.c_str());
    }
    return m;
}

Json povipel_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    Json c = Json::object();
    c.set("vocab", r.integer("vocab", 1));
    c.set("width", r.integer("width", 1));
    c.set("embedding_scale", KeyReader(object_at(raw, "embedding", where), where + ": embedding").number("scale"));
    c.set("norm_eps", KeyReader(object_at(raw, "norm", where), where + ": norm").number("eps"));
    c.set("streams", r.has("streams") ? Json(r.integer("streams", 1)) : Json());
    c.set("logit_softcap", r.has("logit_softcap") ? Json(r.number("logit_softcap", true)) : Json());
    c.set("max_positions", r.integer_or("max_positions", DEFAULT_MAX_POSITIONS, 1));
    if (!raw["layers"].is_array() || raw["layers"].items().empty()) raise(TQE_ERR_CONFIG, "%s: 'layers' must be a list of at least one layer", where.c_str());
    Json list = Json::array();
    long long i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string at = format("%s: layers[%lld]", where.c_str(), i++);
        if (!l.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object", at.c_str());
        const std::string type = KeyReader(l, at).string("type");
        if (type != "parallel" && type != "retention") raise(TQE_ERR_CONFIG, "%s: unknown type '%s' (known: parallel, retention)", at.c_str(), type.c_str());
        Json t = Json::object();
        t.set("type", type);
        t.set("mixer", mixer_typed(object_at(l, "mixer", at), at + ".mixer", type));
        t.set("mlp", mlp_typed(l["mlp"], at + ".mlp"));
        list.push(t);
    }
    c.set("layers", list);
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

ModelSpec povipel_spec(const Json& c) {
    const long long width = c["width"].as_int();
    const Json& eps = c["norm_eps"];
    const Json& max_pos = c["max_positions"];
    const PartSpec norm = part("layer_norm", {{"size", width}, {"eps", eps}, {"tensor", ""}, {"bias_tensor", ".b"}});
    auto rotary = [&](const Json& base, const Json& dims, const char* style) {
        if (dims.as_int() == 0) return Json();          // nothing is turned
        return part("rotary", {{"theta", base}, {"rot_dim", dims}, {"max_positions", max_pos}, {"style", style}}).to_json();
    };
    ModelSpec s;
    s.architecture = "Povipel";
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
        PartSpec mixer;
        if (layer["type"].as_string() == "parallel") {
            const Json& a = m["left"];
            const Json& b = m["right"];
            const PartSpec left = part("pooled_attention", {{"hidden", width}, {"n_heads", a["heads"]}, {"n_kv_heads", a["kv_heads"]}, {"head_dim", a["dim"]},
                {"value_dim", a["vdim"]}, {"scale", a["scale"]}, {"window", a["window"]}, {"pool", a["pool"]}, {"qk_norm", true}, {"eps", eps}, {"sink", true},
                {"rotate_values", true}, {"position", rotary(a["rot_base"], a["rot_dims"], "pairs")}, {"value_position", rotary(a["rot_base"], a["vdim"], "pairs")},
                {"names", names_of({{"q", "q"}, {"k", "k"}, {"v", "v"}, {"o", "o"}, {"q_norm", "q.norm"}, {"k_norm", "k.norm"}, {"sink", "sink"}})}});
            const PartSpec right = part("linear_attention", {{"hidden", width}, {"heads", b["heads"]}, {"head_dim", b["dim"]}, {"value_dim", b["vdim"]},
                {"decay", "channels"}, {"tau", b["tau"]}, {"decay_rank", DEFAULT_DECAY_RANK}, {"q_scale", 1.0 / sqrt((double)b["dim"].as_int())}, {"norm_weight", true},
                {"eps", eps}, {"position", Json()},
                {"names", names_of({{"q", "q"}, {"k", "k"}, {"v", "v"}, {"g", "g"}, {"o", "o"}, {"norm", "norm"}, {"a1", "a1"}, {"a2", "a2"}, {"a2_bias", "a2.b"}})}});
            mixer = part("parallel", {{"hidden", width}, {"first", left.to_json()}, {"second", right.to_json()}, {"eps", eps}, {"scale", PARALLEL_SCALE},
                {"names", names_of({{"first", "left."}, {"second", "right."}, {"first_norm", "left.out"}, {"second_norm", "right.out"}})}});
        } else {
            mixer = part("linear_attention", {{"hidden", width}, {"heads", m["heads"]}, {"head_dim", m["dim"]}, {"value_dim", m["vdim"]}, {"decay", "heads"},
                {"head_decay", m["decay"]}, {"k_scale", 1.0 / sqrt((double)m["dim"].as_int())}, {"norm_weight", false}, {"eps", eps},
                {"position", rotary(m["rot_base"], m["rot_dims"], "halves")},
                {"names", names_of({{"q", "q"}, {"k", "k"}, {"v", "v"}, {"g", "g"}, {"o", "o"}})}});
        }
        Json ff;
        if (!mlp.is_null() && mlp["kind"].as_string() == "dense")
            ff = part("activated", {{"hidden", width}, {"inter", mlp["ff"]}, {"gate", "gelu_tanh"}, {"names", names_of({{"up", "up"}, {"down", "down"}})}}).to_json();
        else if (!mlp.is_null())
            ff = part("routed_experts", {{"hidden", width}, {"inter", mlp["ff"]}, {"n_experts", mlp["experts"]}, {"top", mlp["top"]}, {"router_scale", 1.0},
                {"gate", "silu"}, {"score", "sigmoid"}, {"weight_on", "input"}, {"shared", Json()},
                {"names", names_of({{"router", "router"}, {"expert", "e%d."}, {"gate", "gate"}, {"up", "up"}, {"down", "down"}})}}).to_json();
        LayerSpec spec;
        spec.prefix = format("l%zu.", l++);
        spec.block = part("multi_stream", {{"hidden", width}, {"mixer", mixer.to_json()}, {"feed_forward", ff}, {"mixer_norm", norm.to_json()},
            {"ff_norm", mlp.is_null() ? Json() : norm.to_json()}, {"streams", c["streams"]}, {"token_shift", true},
            {"names", names_of({{"mixer", "mix."}, {"feed_forward", "mlp."}, {"mixer_norm", "norm1"}, {"ff_norm", "norm2"}, {"mixer_streams", "hc1"},
                                {"ff_streams", "hc2"}, {"shift", "shift"}})}});
        s.layers.push_back(spec);
    }
    // the run order: the layers before the span, the span `times` times, the rest
    const long long n = (long long)s.layers.size(), start = c["loop_start"].as_int(), stop = c["loop_stop"].as_int(), times = c["loop_times"].as_int();
    auto run_of = [](long long layer) { Run r; r.layer = (int)layer; return r; };
    for (long long i = 0; i < start; ++i) s.order.push_back(run_of(i));
    for (long long pass = 0; pass < times; ++pass)
        for (long long i = start; i < stop; ++i) s.order.push_back(run_of(i));
    for (long long i = stop; i < n; ++i) s.order.push_back(run_of(i));
    s.final_norm = norm;
    s.final_norm_prefix = "final.norm";
    s.head_name = "head";
    if (!c["logit_softcap"].is_null()) { s.has_logit_cap = true; s.logit_cap = c["logit_softcap"].as_number(); }
    return s;
}

}  // namespace

void register_povipel() {
    Architecture a;
    a.name = "Povipel";
    a.model_types = {"povipel"};
    a.typed_config = povipel_typed;
    a.build_spec = povipel_spec;
    register_architecture(a);
}

}  // namespace tq
