// Attention over a sliding window plus pooled blocks, and a mixer that runs two mixers side by side.
//
//   pooled_attention   grouped-query softmax attention in which position i sees the positions j with 0 <= i - j < window and, for every
//                      block of `pool` positions that lies wholly in front of the window (block b, positions b pool .. b pool + pool - 1,
//                      seen once b pool + pool - 1 <= i - window), one key and one value that are the means of the block's keys and
//                      values as the cache holds them.  Positions that have left the window and whose block is not yet seen are not
//                      seen.  Positions and blocks share one softmax.  Options: qk_norm (q and k heads divided by their root mean
//                      square, times a weight shared by the heads, before the rotation), sink (a learned number per head whose
//                      exponential joins the denominator), rotate_values (a value is turned by its position over all its elements, in
//                      the position part's layout and with angles of its own table, and cached so; a head's output is turned back by
//                      the query's position).  Scores, softmax, norms and angles are float32.
//                      Its pages keep the blocks' means behind the positions: keys [kv heads][page + ceil(page / pool)][head_dim],
//                      values likewise with value_dim; a block lies in the page of its last position.  The cache keeps every page.
//                      params: hidden, n_heads, n_kv_heads, head_dim, value_dim, scale, window, pool, qk_norm, eps, sink,
//                      rotate_values, position (a part spec with tables, or null: q and k are not turned), value_position (a part spec:
//                      the values' tables, whose layout is then the one that counts), names
//                      {q, k, v, o, q_norm, k_norm, sink}.
//   parallel           c (n_a(a(x)) + n_b(b(x))): two mixers read the same input, each output is divided by its root mean square over
//                      the model's width and multiplied by a weight of its own, and the two are added and scaled (c = 1/2).  One of
//                      the two may keep pages and both may keep state: the state rows lie one behind the other in the cache.
//                      params: hidden, first, second (mixer part specs), eps, scale, names {first, second (prefixes), first_norm,
//                      second_norm (tensors)}.
#include <math.h>

#include "kernels.h"
#include "linear.h"
#include "parts.h"
#include "step.h"
#include "trace.h"

namespace tq {
namespace {

OwnedPtr take(Loaded& tensors, const std::string& name) {
    auto it = tensors.find(name);
    if (it == tensors.end() || !it->second) raise(TQE_ERR_WEIGHTS, "a part was not given its tensor '%s'", name.c_str());
    return it->second;
}

OwnedPtr as_floats(const OwnedPtr& p, hipStream_t stream) {
    if (p->t.dtype == F32) return p;
    std::vector<int64_t> dims(p->t.shape, p->t.shape + p->t.ndim);
    OwnedPtr out = make_owned(F32, dims);
    if (!null_device()) K::convert(p->t.data, p->t.dtype, out->t.data, F32, (long long)p->t.numel(), stream);
    stream_synchronize(stream);
    return out;
}

std::shared_ptr<Position> shared_position(const Json& j, const char* what, BuildEnv& env) {
    const PartSpec pos = PartSpec::from_json(j, what);
    const std::string key = "position:" + pos.key();
    auto it = env.shared.find(key);
    if (it == env.shared.end()) it = env.shared.emplace(key, build_part("position", pos, env)).first;
    std::shared_ptr<Position> p = std::dynamic_pointer_cast<Position>(it->second);
    if (!p) raise(TQE_ERR_ARGUMENT, "%s: part kind '%s' is no position", what, pos.kind.c_str());
    if (p->has_apply()) raise(TQE_ERR_ARGUMENT, "%s: the position part must turn from tables", what);
    return p;
}

class PooledAttention : public Mixer {
public:
    PooledAttention(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "pooled_attention", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        n_heads_ = (int)r.integer("n_heads", 1);
        n_kv_heads_ = (int)r.integer("n_kv_heads", 1);
        head_dim_ = (int)r.integer("head_dim", 1);
        value_dim_ = r.has("value_dim") ? (int)r.integer("value_dim", 1) : head_dim_;
        window_ = (int)r.integer("window", 1);
        pool_ = (int)r.integer("pool", 1);
        scale_ = r.has("scale") ? (float)r.number("scale") : (float)(1.0 / sqrt((double)head_dim_));
        qk_norm_ = r.boolean_or("qk_norm", false);
        eps_ = qk_norm_ ? (float)r.number("eps") : 0.f;
        has_sink_ = r.boolean_or("sink", false);
        rotate_values_ = r.boolean_or("rotate_values", false);
        if (n_heads_ % n_kv_heads_) raise(TQE_ERR_ARGUMENT, "pooled_attention: %d heads are not a multiple of %d kv heads", n_heads_, n_kv_heads_);
        const int most = K::pooled_attention_max_dim.raw();
        if (head_dim_ > most || value_dim_ > most)
            raise(TQE_ERR_CONFIG, "pooled_attention: heads of %d and %d values are more than the attention kernels take (%d)", head_dim_, value_dim_, most);
        const Json& names = spec.params["names"];
        auto name = [&](const char* role, const char* fallback) { return names[role].is_string() ? names[role].as_string() : std::string(fallback); };
        n_q_ = name("q", "q_proj.weight"); n_k_ = name("k", "k_proj.weight"); n_v_ = name("v", "v_proj.weight"); n_o_ = name("o", "o_proj.weight");
        n_q_norm_ = name("q_norm", "q_norm.weight"); n_k_norm_ = name("k_norm", "k_norm.weight"); n_sink_ = name("sink", "sink");
        if (!spec.params["position"].is_null()) position_ = shared_position(spec.params["position"], "pooled_attention: position", env);
        if (position_ && position_->tables().rot_dim > head_dim_) raise(TQE_ERR_ARGUMENT, "pooled_attention: %d turned elements in heads of %d", position_->tables().rot_dim, head_dim_);
        if (rotate_values_) {
            value_position_ = shared_position(spec.params["value_position"], "pooled_attention: value_position", env);
            const Position::Tables vt = value_position_->tables();
            if (vt.rot_dim != value_dim_ || vt.style == STYLE_NONE || (position_ && position_->tables().style != STYLE_NONE && position_->tables().style != vt.style))
                raise(TQE_ERR_ARGUMENT, "pooled_attention: values are turned over all their %d elements, in the layout of the keys", value_dim_);
        }
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        const int64_t q = (int64_t)n_heads_ * head_dim_, kv = (int64_t)n_kv_heads_ * head_dim_;
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        TensorSpecs t = {{n_q_, w(q, hidden_)}, {n_k_, w(kv, hidden_)}, {n_v_, w((int64_t)n_kv_heads_ * value_dim_, hidden_)},
                         {n_o_, w(hidden_, (int64_t)n_heads_ * value_dim_)}};
        if (qk_norm_) {
            TensorSpec n; n.shape = {head_dim_}; n.init = "one_plus_normal"; n.std_dev = 0.1;
            t.push_back({n_q_norm_, n});
            t.push_back({n_k_norm_, n});
        }
        if (has_sink_) { TensorSpec s; s.shape = {n_heads_}; s.std_dev = 1.0; t.push_back({n_sink_, s}); }
        return t;
    }
    void load(Loaded& t, hipStream_t stream) override {
        w_qkv_ = make_weight(stack_rows({take(t, n_q_), take(t, n_k_), take(t, n_v_)}, stream), 1, false, stream);
        w_o_ = make_weight(take(t, n_o_), 1, false, stream);
        if (qk_norm_) { q_norm_ = as_floats(take(t, n_q_norm_), stream); k_norm_ = as_floats(take(t, n_k_norm_), stream); }
        if (has_sink_) sink_ = as_floats(take(t, n_sink_), stream);
        stored_ = t;
        for (const std::string& big : {n_q_, n_k_, n_v_, n_o_}) stored_.erase(big);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "qkv.weight") return w_qkv_.rows;
        if (name == "o.weight") return w_o_.rows;
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    const char* trace_name() const override { return "attn"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({(int64_t)(n_heads_ + n_kv_heads_) * head_dim_ + (int64_t)n_kv_heads_ * value_dim_, hidden_});
        out.push_back({hidden_, (int64_t)n_heads_ * value_dim_});
    }
    CacheNeed cache_need() const override {
        const int rows = TQE_PAGE + K::pooled_rows.raw(pool_);
        CacheNeed n;
        n.kind = CacheNeed::Pages;
        n.key_page = {n_kv_heads_, rows, head_dim_};
        n.value_page = {n_kv_heads_, rows, value_dim_};
        return n;
    }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (!entry.keys.defined() || !entry.writes) raise(TQE_ERR_STATE, "pooled_attention was given no pages of its own in the cache");
        if (last_rows || x.lazy || stream) raise(TQE_ERR_STATE, "pooled_attention takes all rows of the step, as they are, and returns its output");
        const int64_t n = x.x.shape[0];
        const int dtype = x.x.dtype;
        if (entry.keys.dtype != dtype) raise(TQE_ERR_STATE, "pooled_attention: the cache holds %s, the step runs in %s", dtype_name(entry.keys.dtype), dtype_name(dtype));
        const StepContext::Table& table = c.tables.at((size_t)entry.group);
        const Tensor qkv = linear(c, x.x, w_qkv_, nullptr, dtype).t;
        Position::Tables tb, vt;
        if (position_) tb = position_->tables();
        if (rotate_values_) vt = value_position_->tables();
        const bool turn = tb.style != STYLE_NONE;
        const int style = rotate_values_ ? vt.style : tb.style;
        const int max_pos = rotate_values_ && turn ? (int)std::min(tb.cos.shape[0], vt.cos.shape[0]) : rotate_values_ ? (int)vt.cos.shape[0] : turn ? (int)tb.cos.shape[0] : 1 << 30;
        const float* vcos = rotate_values_ ? (const float*)vt.cos.data : nullptr;
        const float* vsin = rotate_values_ ? (const float*)vt.sin.data : nullptr;
        Tensor q = c.alloc(dtype, {n, n_heads_, head_dim_});
        K::pooled_store(qkv.data, dtype, qk_norm_ ? (const float*)q_norm_->t.data : nullptr, qk_norm_ ? (const float*)k_norm_->t.data : nullptr, qk_norm_ ? 1 : 0, eps_,
                        turn ? (const float*)tb.cos.data : nullptr, turn ? (const float*)tb.sin.data : nullptr, turn ? tb.rot_dim : 0, style, vcos, vsin, max_pos,
                        c.dev.tok_seq, c.dev.tok_pos, table.dev, table.width, entry.keys.data, entry.values.data, q.data, (int)n, n_heads_, n_kv_heads_, head_dim_,
                        value_dim_, pool_, c.stream);
        K::pool_blocks(entry.keys.data, entry.values.data, dtype, c.dev.seq_start, c.dev.seq_new, table.dev, table.width, c.n_seqs, c.max_new, pool_, n_kv_heads_,
                       head_dim_, value_dim_, c.stream);
        Tensor y = c.alloc(dtype, {n, (int64_t)n_heads_ * value_dim_});
        // bfloat16 steps that bring several tokens of a sequence: tiles of consecutive queries on the matrix cores, where the heads' sizes
        // allow; steps of one token a sequence, the 32-bit path and other sizes: the plain kernel, a wave per (row, head)
        if (dtype == BF16 && !c.all_decode && !c.capturing && policy().prefill_mfma && !null_device() &&
            K::pooled_attention_tiles_supported.raw(head_dim_, value_dim_)) {
            const int tile = K::pooled_attention_tile.raw(n_heads_, n_kv_heads_);
            const Tiles t = c.query_tiles(tile);
            K::pooled_attention_tiles(q.data, entry.keys.data, entry.values.data, c.dev.tok_pos, table.dev, table.width, window_, pool_, scale_,
                                      has_sink_ ? (const float*)sink_->t.data : nullptr, vcos, vsin, style, max_pos, t.seq, t.tok0, t.count, t.n, tile, y.data,
                                      n_heads_, n_kv_heads_, head_dim_, value_dim_, c.stream);
            return linear(c, y, w_o_, nullptr, dtype).t;
        }
        K::pooled_attention(q.data, entry.keys.data, entry.values.data, dtype, c.dev.tok_seq, c.dev.tok_pos, table.dev, table.width, window_, pool_, scale_,
                            has_sink_ ? (const float*)sink_->t.data : nullptr, vcos, vsin, style, max_pos, y.data, (int)n, n_heads_, n_kv_heads_, head_dim_,
                            value_dim_, c.stream);
        return linear(c, y, w_o_, nullptr, dtype).t;
    }

private:
    int64_t hidden_;
    int n_heads_, n_kv_heads_, head_dim_, value_dim_, window_, pool_;
    float scale_, eps_;
    bool qk_norm_, has_sink_, rotate_values_;
    std::string n_q_, n_k_, n_v_, n_o_, n_q_norm_, n_k_norm_, n_sink_;
    std::shared_ptr<Position> position_, value_position_;
    Weight w_qkv_, w_o_;
    OwnedPtr q_norm_, k_norm_, sink_;
    Loaded stored_;
};

class ParallelMixer : public Mixer {
public:
    ParallelMixer(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "parallel", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        eps_ = (float)r.number("eps");
        scale_ = (float)r.number_or("scale", 0.5);
        const Json& names = spec.params["names"];
        auto name = [&](const char* role, const char* fallback) { return names[role].is_string() ? names[role].as_string() : std::string(fallback); };
        prefix_[0] = name("first", "first."); prefix_[1] = name("second", "second.");
        n_norm_[0] = name("first_norm", "first.norm"); n_norm_[1] = name("second_norm", "second.norm");
        const char* roles[2] = {"first", "second"};
        for (int i = 0; i < 2; ++i) {
            part_[i] = std::dynamic_pointer_cast<Mixer>(build_part("mixer", PartSpec::from_json(spec.params[roles[i]], roles[i]), env));
            if (!part_[i]) raise(TQE_ERR_ARGUMENT, "parallel: '%s' is no mixer", roles[i]);
            need_[i] = part_[i]->cache_need();
            state_len_[i] = 0;
            if (need_[i].has_state()) {
                if (need_[i].state_dtype != F32) raise(TQE_ERR_ARGUMENT, "parallel: the state of '%s' is not float32", roles[i]);
                state_len_[i] = 1;
                for (int64_t v : need_[i].state_shape) state_len_[i] *= v;
            }
        }
        if (need_[0].kind == CacheNeed::Pages && need_[1].kind == CacheNeed::Pages) raise(TQE_ERR_ARGUMENT, "parallel: both mixers keep pages, the cache gives a run one kind");
        graph_safe = part_[0]->graph_safe && part_[1]->graph_safe;
    }
    TensorSpecs tensors() const override {
        TensorSpecs out;
        for (int i = 0; i < 2; ++i) {
            for (const auto& t : part_[i]->tensors()) out.push_back({prefix_[i] + t.first, t.second});
            TensorSpec n; n.shape = {hidden_}; n.init = "one_plus_normal"; n.std_dev = 0.1;
            out.push_back({n_norm_[i], n});
        }
        return out;
    }
    void load(Loaded& tensors, hipStream_t stream) override {
        for (int i = 0; i < 2; ++i) {
            Loaded own;
            for (const auto& t : part_[i]->tensors()) own[t.first] = take(tensors, prefix_[i] + t.first);
            part_[i]->load(own, stream);
            norm_w_[i] = as_floats(take(tensors, n_norm_[i]), stream);
            stored_[n_norm_[i]] = take(tensors, n_norm_[i]);
        }
    }
    OwnedPtr held(const std::string& name) const override {
        for (int i = 0; i < 2; ++i)
            if (name.compare(0, prefix_[i].size(), prefix_[i]) == 0)
                if (OwnedPtr p = part_[i]->held(name.substr(prefix_[i].size()))) return p;
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    Json describe() const override {
        Json j = Part::describe();
        Json parts = Json::object();
        parts.set("first", part_[0]->describe());
        parts.set("second", part_[1]->describe());
        j.set("parts", parts);
        return j;
    }
    const char* trace_name() const override { return "attn"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        for (int i = 0; i < 2; ++i) part_[i]->product_shapes(out);
    }
    // the pages of the one that keeps pages; the two states one behind the other
    CacheNeed cache_need() const override {
        CacheNeed n = need_[0].kind == CacheNeed::Pages ? need_[0] : need_[1].kind == CacheNeed::Pages ? need_[1] : CacheNeed();
        n.state_shape.clear();
        if (state_len_[0] + state_len_[1] > 0) {
            if (n.kind == CacheNeed::None) n.kind = CacheNeed::State;
            n.state_shape = {state_len_[0] + state_len_[1]};
            n.state_dtype = F32;
        }
        return n;
    }
    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (last_rows || x.lazy || stream) raise(TQE_ERR_STATE, "parallel takes all rows of the step, as they are, and returns its output");
        Tensor y[2];
        for (int i = 0; i < 2; ++i) {
            CacheEntry own = entry;
            own.kind = need_[i].kind;
            if (need_[i].kind != CacheNeed::Pages) { own.keys = Tensor(); own.values = Tensor(); own.group = -1; }
            if (state_len_[i] == 0) own.state = Tensor();
            else own.state_offset = entry.state_offset + (i == 1 ? state_len_[0] : 0);
            Span span(part_[i]->trace_name());
            y[i] = part_[i]->forward(c, x, own, nullptr, false);
        }
        if (y[0].dtype != y[1].dtype || y[0].shape[0] != y[1].shape[0] || y[0].cols() != hidden_ || y[1].cols() != hidden_)
            raise(TQE_ERR_STATE, "parallel: the two mixers returned %s and %s", y[0].describe().c_str(), y[1].describe().c_str());
        Tensor out = c.alloc(y[0].dtype, {y[0].shape[0], hidden_});
        K::normed_pair_sum(y[0].data, y[1].data, y[0].dtype, (const float*)norm_w_[0]->t.data, (const float*)norm_w_[1]->t.data, eps_, scale_, out.data, out.dtype,
                           (int)y[0].shape[0], (int)hidden_, c.stream);
        return out;
    }

private:
    int64_t hidden_, state_len_[2];
    float eps_, scale_;
    std::string prefix_[2], n_norm_[2];
    std::shared_ptr<Mixer> part_[2];
    CacheNeed need_[2];
    OwnedPtr norm_w_[2];
    Loaded stored_;
};

}  // namespace

void register_pooled_parts() {
    register_kind("mixer", "pooled_attention", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<PooledAttention>(s, e); });
    register_kind("mixer", "parallel", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<ParallelMixer>(s, e); });
}

}  // namespace tq
