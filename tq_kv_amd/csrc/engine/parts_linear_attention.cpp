// A mixer of linear attention with a decaying state instead of keys and values.
//
//   linear_attention   per head S_t = diag(a_t) S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with q, k of head_dim and v of value_dim
//                      elements, no softmax and no denominator.  The decay is
//                        decay "heads":     one fixed number per head (head_decay, a list), the retention form; or
//                        decay "channels":  one number per key channel and token, a = sigmoid(W_a2 (W_a1 x) + b)^(1/tau), through a
//                                           product of low rank whose rank the checkpoint's tensors give.
//                      q and k may be turned by the position (a position part with tables, over the first rot_dim elements, in the
//                      part's layout) and are multiplied by q_scale and k_scale after that.  Each head's output is divided by its
//                      root mean square (times a weight over the head's elements if norm_weight), the heads side by side are
//                      multiplied by silu(W_g x), and W_o projects back.
//
// The state, [heads][head_dim][value_dim] float32 per sequence, is a row of the cache's state groups (zero when a slot is taken).
// Decays, their logarithms, the state and the heads' norm are float32 whatever the activation type; the products are the
// framework's (linear.cpp), q, k, v and the gate as one product with the weights stacked.  Steps that bring many tokens of a sequence
// run the recurrence in chunks (every chunk from a zero state, a carry over the chunks, every chunk again with the outputs).
//
// params: hidden, heads, head_dim, value_dim, decay ("heads" | "channels"), head_decay (list, for "heads"), tau and decay_rank (for
// "channels"; decay_rank is what random weights get), q_scale, k_scale (1 unless given), norm_weight, eps, position (a part spec, or
// null), names {q, k, v, g, o, norm, a1, a2, a2_bias}.
#include <math.h>

#include "kernels.h"
#include "linear.h"
#include "parts.h"
#include "step.h"

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

const void* at(const Tensor& t, int64_t column) { return (const char*)t.data + (size_t)column * dtype_size(t.dtype); }

class LinearAttention : public Mixer {
public:
    LinearAttention(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "linear_attention", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        heads_ = (int)r.integer("heads", 1);
        d_ = (int)r.integer("head_dim", 1);
        dv_ = (int)r.integer("value_dim", 1);
        const std::string decay = r.string("decay");
        if (decay == "heads") per_channel_ = false;
        else if (decay == "channels") per_channel_ = true;
        else raise(TQE_ERR_ARGUMENT, "linear_attention: unknown decay '%s' (known: channels, heads)", decay.c_str());
        if (per_channel_) {
            tau_ = r.number("tau", true);
            rank_ = r.integer_or("decay_rank", 16, 1);
        } else {
            const Json& list = spec.params["head_decay"];
            if (!list.is_array() || (int)list.items().size() != heads_) raise(TQE_ERR_ARGUMENT, "linear_attention: head_decay must list one number for each of the %d heads", heads_);
            for (const Json& v : list.items()) {
                if (!v.is_number()) raise(TQE_ERR_ARGUMENT, "linear_attention: head_decay holds something that is no number");
                head_decay_.push_back((float)v.as_number());
            }
        }
        q_scale_ = (float)r.number_or("q_scale", 1.0);
        k_scale_ = (float)r.number_or("k_scale", 1.0);
        norm_weight_ = r.boolean_or("norm_weight", false);
        eps_ = (float)r.number("eps");
        if (d_ > K::linear_attention_max_dim.raw()) raise(TQE_ERR_CONFIG, "linear_attention: heads of %d key channels are more than the kernels take (%d)", d_, K::linear_attention_max_dim.raw());
        const Json& n = spec.params["names"];
        auto name = [&](const char* role, const char* fallback) { return n[role].is_string() ? n[role].as_string() : std::string(fallback); };
        n_q_ = name("q", "q"); n_k_ = name("k", "k"); n_v_ = name("v", "v"); n_g_ = name("g", "g"); n_o_ = name("o", "o"); n_norm_ = name("norm", "norm");
        n_a1_ = name("a1", "a1"); n_a2_ = name("a2", "a2"); n_a2b_ = name("a2_bias", "a2.bias");
        graph_safe = true;
        if (!spec.params["position"].is_null()) {
            const PartSpec pos = PartSpec::from_json(spec.params["position"], "linear_attention: position");
            const std::string key = "position:" + pos.key();
            auto it = env.shared.find(key);
            if (it == env.shared.end()) it = env.shared.emplace(key, build_part("position", pos, env)).first;
            position_ = std::dynamic_pointer_cast<Position>(it->second);
            if (!position_) raise(TQE_ERR_ARGUMENT, "linear_attention: part kind '%s' is no position", pos.kind.c_str());
            if (position_->has_apply()) raise(TQE_ERR_ARGUMENT, "linear_attention: the position part must turn from tables");
            if (position_->tables().rot_dim > d_) raise(TQE_ERR_ARGUMENT, "linear_attention: %d turned elements in heads of %d", position_->tables().rot_dim, d_);
        }
    }
    TensorSpecs tensors() const override {
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        const int64_t qk = (int64_t)heads_ * d_, vv = (int64_t)heads_ * dv_;
        TensorSpecs t = {{n_q_, w(qk, hidden_)}, {n_k_, w(qk, hidden_)}, {n_v_, w(vv, hidden_)}, {n_g_, w(vv, hidden_)}, {n_o_, w(hidden_, vv)}};
        if (norm_weight_) { TensorSpec n; n.shape = {dv_}; n.init = "one_plus_normal"; n.std_dev = 0.1; t.push_back({n_norm_, n}); }
        if (per_channel_) {
            TensorSpec a1 = w(rank_, hidden_); a1.free = {0};
            TensorSpec a2 = w(qk, rank_); a2.free = {1}; a2.std_dev = 0.5;
            TensorSpec b; b.shape = {qk}; b.std_dev = 1.0;
            t.push_back({n_a1_, a1});
            t.push_back({n_a2_, a2});
            t.push_back({n_a2b_, b});
        }
        return t;
    }
    void load(Loaded& t, hipStream_t stream) override {
        // (rows up to a multiple of 16, so that the product's rows stay at multiples of 16 bytes whatever the sizes)
        OwnedPtr in = stack_rows({take(t, n_q_), take(t, n_k_), take(t, n_v_), take(t, n_g_)}, stream, 16);
        row_ = in->t.shape[0];
        w_in_ = make_weight(in, 1, false, stream);
        w_o_ = make_weight(take(t, n_o_), 1, false, stream);
        if (norm_weight_) norm_w_ = as_floats(take(t, n_norm_), stream);
        if (per_channel_) {
            OwnedPtr a1 = take(t, n_a1_), a2 = take(t, n_a2_);
            if (a1->t.shape[0] != a2->t.shape[1])
                raise(TQE_ERR_WEIGHTS, "linear_attention: the decay's two matrices do not meet: %s and %s", a1->t.describe().c_str(), a2->t.describe().c_str());
            w_a1_ = make_weight(a1, 1, false, stream);
            w_a2_ = make_weight(a2, 1, false, stream);
            a2_bias_ = as_floats(take(t, n_a2b_), stream);
        } else {
            decay_ = make_owned(F32, {(int64_t)heads_});
            copy_to_device(decay_->t.data, head_decay_.data(), head_decay_.size() * 4, stream);
            stream_synchronize(stream);
        }
        stored_ = t;
        for (const std::string& big : {n_q_, n_k_, n_v_, n_g_, n_o_, n_a1_, n_a2_}) stored_.erase(big);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "in.weight") return w_in_.rows;
        if (name == "o.weight") return w_o_.rows;
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    const char* trace_name() const override { return "linear-attn"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({(2LL * heads_ * d_ + 2LL * heads_ * dv_ + 15) / 16 * 16, hidden_});
        out.push_back({hidden_, (int64_t)heads_ * dv_});
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::State;
        n.state_shape = {(int64_t)heads_ * d_ * dv_};
        n.state_dtype = F32;
        return n;
    }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (!entry.state.defined() || !entry.writes) raise(TQE_ERR_STATE, "linear_attention was given no state of its own in the cache");
        if (last_rows || x.lazy || stream) raise(TQE_ERR_STATE, "linear_attention takes all rows of the step, as they are, and returns its output");
        const int64_t n = x.x.shape[0];
        const int dtype = x.x.dtype;
        const long long row = entry.state.cols();
        float* state = (float*)entry.state.data + entry.state_offset;
        const int64_t qk = (int64_t)heads_ * d_, vv = (int64_t)heads_ * dv_;
        const Tensor in = linear(c, x.x, w_in_, nullptr, dtype).t;                    // [q | k | v | g | padding]
        Tensor z;
        if (per_channel_) {
            const Tensor low = linear(c, x.x, w_a1_, nullptr, dtype).t;
            z = linear(c, low, w_a2_, nullptr, F32).t;
        }
        Position::Tables tb;
        if (position_) tb = position_->tables();
        const bool turn = tb.style != STYLE_NONE;
        const float* cos = turn ? (const float*)tb.cos.data : nullptr;
        const float* sin = turn ? (const float*)tb.sin.data : nullptr;
        const int max_pos = turn ? (int)tb.cos.shape[0] : 0;
        const float* zp = per_channel_ ? (const float*)z.data : nullptr;
        const float* zb = per_channel_ ? (const float*)a2_bias_->t.data : nullptr;
        const float* hd = per_channel_ ? nullptr : (const float*)decay_->t.data;
        const float inv_tau = per_channel_ ? (float)(1.0 / tau_) : 0.f;
        Tensor o = c.alloc(F32, {n, heads_, dv_});
        auto run = [&](int mode, int items, const Chunks* ch, float* cs, float* cd) {
            K::linear_attention(in.data, at(in, qk), at(in, 2 * qk), dtype, row_, zp, qk, zb, inv_tau, hd, q_scale_, k_scale_, cos, sin, turn ? tb.rot_dim : 0,
                                turn ? tb.style : 0, max_pos, c.dev.tok_pos, state, row, c.dev.cu, c.dev.seq_new, c.dev.seq_slot, ch ? ch->row0 : nullptr,
                                ch ? ch->count : nullptr, cs, cd, (float*)o.data, mode, items, heads_, d_, dv_, c.stream);
        };
        if (dtype == BF16 && !c.all_decode && !c.capturing && c.max_new >= CHUNKED_FROM && !null_device()) {
            const Chunks ch = c.chunks(SCAN_CHUNK);
            const int64_t per_seq = qk * dv_;
            Tensor cs = c.alloc(F32, {ch.n, per_seq}), cd = c.alloc(F32, {ch.n, qk});
            run(1, ch.n, &ch, (float*)cs.data, (float*)cd.data);
            K::chunk_carry((const float*)cd.data, qk, dv_, (float*)cs.data, ch.seq_first, c.dev.seq_slot, state, row, c.n_seqs, per_seq, c.stream);
            run(2, ch.n, &ch, (float*)cs.data, (float*)cd.data);
        } else {
            run(0, c.n_seqs, nullptr, nullptr, nullptr);
        }
        Tensor gated = c.alloc(dtype, {n, vv});
        K::head_norm_gate((const float*)o.data, norm_w_ ? (const float*)norm_w_->t.data : nullptr, eps_, at(in, 2 * qk + vv), dtype, row_, gated.data, dtype, (int)n,
                          heads_, dv_, c.stream);
        return linear(c, gated, w_o_, nullptr, dtype).t;
    }

private:
    static const int CHUNKED_FROM = 128, SCAN_CHUNK = 64;
    int64_t hidden_, row_ = 0, rank_ = 16;
    int heads_, d_, dv_;
    bool per_channel_ = false, norm_weight_ = false;
    double tau_ = 1.0;
    float q_scale_ = 1.f, k_scale_ = 1.f, eps_ = 0.f;
    std::vector<float> head_decay_;
    std::string n_q_, n_k_, n_v_, n_g_, n_o_, n_norm_, n_a1_, n_a2_, n_a2b_;
    std::shared_ptr<Position> position_;
    Weight w_in_, w_o_, w_a1_, w_a2_;
    OwnedPtr norm_w_, a2_bias_, decay_;
    Loaded stored_;
};

}  // namespace

void register_linear_attention_parts() {
    register_kind("mixer", "linear_attention", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<LinearAttention>(s, e); });
}

}  // namespace tq
