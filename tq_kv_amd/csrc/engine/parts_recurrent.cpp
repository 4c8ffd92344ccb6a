// Mixers that keep a fixed-size state per sequence instead of keys and values.
//
//   rglru    the recurrent block of the Griffin family: two branches of `width` channels, y = gelu_tanh(W_y h + b_y) and
//            u = conv(W_x h + b_x) (a short causal convolution per channel); gates r = sigmoid(W_a u + b_a), i = sigmoid(W_i u + b_i)
//            with block-diagonal W_a, W_i; a = exp(-decay_scale r softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) i u; output W_o (S y).
//   mamba2   the selective state-space mixer with a scalar decay per head: one product gives [z | x | B | C | dt]; x, B, C pass a short
//            causal convolution and SiLU; dt = softplus(dt + dt_bias); per head S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T,
//            y_t = S_t^T C_t + D x_t; y silu(z) is normed in `norm_groups` equal parts, times a weight, then W_o.
//
// Both keep, per sequence, the convolution's last taps - 1 inputs and the recurrence's state, in float32, as one row of the cache's
// state groups (zero when a slot is taken): [conv inputs (taps - 1) x channels | state].  Everything that enters a recurrence is
// computed in float32 whatever the activation type; the products are the framework's (linear.cpp).  Sizes, the convolution's
// length, the decay's scale and every tensor's name are parameters.
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

// a small tensor's values on the host, as float32
std::vector<float> host_floats(const OwnedPtr& p, hipStream_t stream) {
    const Tensor& t = p->t;
    std::vector<float> out((size_t)t.numel());
    if (t.dtype == F32) copy_to_host(out.data(), t.data, t.bytes(), stream);
    else {
        std::vector<uint16_t> bits((size_t)t.numel());
        copy_to_host(bits.data(), t.data, t.bytes(), stream);
        for (size_t i = 0; i < bits.size(); ++i) {
            const uint32_t u = (uint32_t)bits[i] << 16;
            memcpy(&out[i], &u, 4);
        }
    }
    return out;
}

OwnedPtr device_floats(const std::vector<float>& v, hipStream_t stream) {
    OwnedPtr p = make_owned(F32, {(int64_t)v.size()});
    copy_to_device(p->t.data, v.data(), v.size() * 4, stream);
    stream_synchronize(stream);
    return p;
}

OwnedPtr as_floats(const OwnedPtr& p, hipStream_t stream) { return p->t.dtype == F32 ? p : device_floats(host_floats(p, stream), stream); }

std::string name_of(const Json& names, const char* role, const char* fallback) {
    return names[role].is_string() ? names[role].as_string() : std::string(fallback);
}

TensorSpec matrix(int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; }
TensorSpec vector_of(int64_t a, double std_dev = 0.02) { TensorSpec t; t.shape = {a}; t.std_dev = std_dev; return t; }

// Steps that bring so many tokens of some sequence run their recurrences in chunks (three launches, every chunk a piece of work of its
// own); shorter ones, steps of one token a sequence and the 32-bit path run them token by token, where the order of the sums does not
// depend on how a sequence was cut.
const int CHUNKED_FROM = 128;
bool in_chunks(const StepContext& c, int dtype) { return dtype == BF16 && !c.all_decode && !c.capturing && c.max_new >= CHUNKED_FROM && !null_device(); }

const void* at(const Tensor& t, int64_t column) { return (const char*)t.data + (size_t)column * dtype_size(t.dtype); }

// ---- rglru -------------------------------------------------------------------------------------------
// params: hidden, width, blocks, conv (taps); optional decay_scale (8 unless given), names {y, y_bias, x, x_bias, conv, conv_bias,
// gate_a, gate_a_bias, gate_i, gate_i_bias, decay, o}.
class RGLRU : public Mixer {
public:
    RGLRU(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "rglru", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        width_ = r.integer("width", 1);
        blocks_ = (int)r.integer("blocks", 1);
        taps_ = (int)r.integer("conv", 1);
        decay_scale_ = r.number_or("decay_scale", 8.0, true);
        if (width_ % blocks_) raise(TQE_ERR_CONFIG, "rglru: a width of %lld does not fall into %d blocks", (long long)width_, blocks_);
        if (taps_ > K::conv_max_taps.raw()) raise(TQE_ERR_CONFIG, "rglru: a convolution of %d taps is more than the kernels take (%d)", taps_, K::conv_max_taps.raw());
        if (width_ / blocks_ > 2048) raise(TQE_ERR_CONFIG, "rglru: gate blocks of %lld channels are more than the kernels take (2048)", (long long)(width_ / blocks_));
        const Json& n = spec.params["names"];
        n_y_ = name_of(n, "y", "y.weight"); n_yb_ = name_of(n, "y_bias", "y.bias"); n_x_ = name_of(n, "x", "x.weight"); n_xb_ = name_of(n, "x_bias", "x.bias");
        n_conv_ = name_of(n, "conv", "conv.weight"); n_convb_ = name_of(n, "conv_bias", "conv.bias");
        n_a_ = name_of(n, "gate_a", "gate_a.weight"); n_ab_ = name_of(n, "gate_a_bias", "gate_a.bias");
        n_i_ = name_of(n, "gate_i", "gate_i.weight"); n_ib_ = name_of(n, "gate_i_bias", "gate_i.bias");
        n_decay_ = name_of(n, "decay", "decay"); n_o_ = name_of(n, "o", "o.weight");
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        const int64_t bs = width_ / blocks_;
        TensorSpec gate; gate.shape = {blocks_, bs, bs}; gate.std_dev = 0.1;
        TensorSpec gate_bias; gate_bias.shape = {blocks_, bs}; gate_bias.std_dev = 0.5;
        TensorSpec conv = matrix(width_, taps_); conv.std_dev = 0.3;
        return {{n_y_, matrix(width_, hidden_)}, {n_yb_, vector_of(width_, 0.1)}, {n_x_, matrix(width_, hidden_)}, {n_xb_, vector_of(width_, 0.1)},
                {n_conv_, conv}, {n_convb_, vector_of(width_, 0.1)}, {n_a_, gate}, {n_ab_, gate_bias}, {n_i_, gate}, {n_ib_, gate_bias},
                {n_decay_, vector_of(width_, 1.0)}, {n_o_, matrix(hidden_, width_)}};
    }
    void load(Loaded& t, hipStream_t stream) override {
        w_yx_ = make_weight(stack_rows({take(t, n_y_), take(t, n_x_)}, stream), 1, false, stream);
        w_o_ = make_weight(take(t, n_o_), 1, false, stream);
        y_bias_ = as_floats(take(t, n_yb_), stream);
        x_bias_ = as_floats(take(t, n_xb_), stream);
        conv_w_ = as_floats(take(t, n_conv_), stream);
        conv_b_ = as_floats(take(t, n_convb_), stream);
        gate_a_b_ = as_floats(take(t, n_ab_), stream);
        gate_i_b_ = as_floats(take(t, n_ib_), stream);
        // the gates' matrices with the input index first, in float32 (small: width^2 / blocks values each)
        const int64_t bs = width_ / blocks_;
        auto turned = [&](const OwnedPtr& p) {
            const std::vector<float> w = host_floats(p, stream);
            std::vector<float> out(w.size());
            for (int64_t b = 0; b < blocks_; ++b)
                for (int64_t o = 0; o < bs; ++o)
                    for (int64_t i = 0; i < bs; ++i) out[(size_t)((b * bs + i) * bs + o)] = w[(size_t)((b * bs + o) * bs + i)];
            return device_floats(out, stream);
        };
        gate_a_ = turned(take(t, n_a_));
        gate_i_ = turned(take(t, n_i_));
        // log a = decay_c r with decay_c = -decay_scale softplus(lam)
        std::vector<float> lam = host_floats(take(t, n_decay_), stream);
        for (float& v : lam) v = (float)(-decay_scale_ * (v > 30.f ? (double)v : log1p(exp((double)v))));
        decay_c_ = device_floats(lam, stream);
        stored_ = t;
        for (const std::string& big : {n_y_, n_x_, n_o_}) stored_.erase(big);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "yx.weight") return w_yx_.rows;
        if (name == "o.weight") return w_o_.rows;
        if (name == "decay.effective") return decay_c_;
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    const char* trace_name() const override { return "rglru"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({2 * width_, hidden_});
        out.push_back({hidden_, width_});
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::State;
        n.state_shape = {(int64_t)(taps_ - 1) * width_ + width_};
        n.state_dtype = F32;
        return n;
    }
    bool adds_to_stream(const StepContext& c) const override { return fusable(c.n_tokens, w_o_, true) || leaves_sums(c.n_tokens, w_o_); }
    // (steps of few rows: the first product divides by the rows' root mean square itself)
    bool folds_norm(const StepContext& c) const override { return fusable(c.n_tokens, w_yx_); }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (entry.kind != CacheNeed::State || !entry.writes) raise(TQE_ERR_STATE, "rglru was given no state of its own in the cache");
        if (last_rows) raise(TQE_ERR_STATE, "rglru takes all rows of the step");
        const int64_t n = x.rows();
        const int dtype = x.lazy ? BF16 : x.x.dtype;
        const long long row = entry.state.cols(), conv_part = (long long)(taps_ - 1) * width_;
        float* state = (float*)entry.state.data + entry.state_offset;
        const Tensor yx = x.lazy ? linear_of_norm(c, x.norm, w_yx_, dtype) : linear(c, x.x, w_yx_, nullptr, dtype).t;
        Tensor u = c.alloc(F32, {n, width_}), a = c.alloc(F32, {n, width_}), g = c.alloc(F32, {n, width_});
        if (c.all_decode) {
            K::conv_state_step(at(yx, width_), dtype, 2 * width_, (const float*)x_bias_->t.data, (const float*)conv_w_->t.data, (const float*)conv_b_->t.data,
                               taps_, 0, state, row, c.dev.tok_seq, c.dev.seq_slot, (float*)u.data, (int)n, (int)width_, c.stream);
        } else {
            K::conv_state(at(yx, width_), dtype, 2 * width_, (const float*)x_bias_->t.data, (const float*)conv_w_->t.data, (const float*)conv_b_->t.data, taps_, 0,
                          state, row, c.dev.tok_seq, c.dev.tok_pos, c.dev.seq_slot, c.dev.seq_start, (float*)u.data, (int)n, (int)width_, c.stream);
            K::conv_state_update(at(yx, width_), dtype, 2 * width_, (const float*)x_bias_->t.data, taps_, state, row, c.dev.cu, c.dev.seq_new, c.dev.seq_slot,
                                 c.n_seqs, (int)width_, c.stream);
        }
        // (32-bit steps keep one order of the gates' sums whatever the step holds)
        (dtype == BF16 ? K::rglru_gates_any_order : K::rglru_gates)(
            (const float*)u.data, (const float*)gate_a_->t.data, (const float*)gate_i_->t.data, (const float*)gate_a_b_->t.data,
            (const float*)gate_i_b_->t.data, (const float*)decay_c_->t.data, (float*)a.data, (float*)g.data, (int)n, (int)width_, blocks_, c.stream);
        Tensor out = c.alloc(dtype, {n, width_});
        if (in_chunks(c, dtype)) {
            const Chunks ch = c.chunks(SCAN_CHUNK);
            Tensor cp = c.alloc(F32, {ch.n, width_}), cl = c.alloc(F32, {ch.n, width_});
            K::linear_chunks((const float*)a.data, (const float*)g.data, nullptr, dtype, 0, nullptr, ch.row0, ch.count, ch.n, (float*)cp.data, (float*)cl.data,
                             nullptr, 1, (int)width_, c.stream);
            K::chunk_carry((const float*)cp.data, width_, 1, (float*)cl.data, ch.seq_first, c.dev.seq_slot, state + conv_part, row, c.n_seqs, width_, c.stream);
            K::linear_chunks((const float*)a.data, (const float*)g.data, yx.data, dtype, 2 * width_, (const float*)y_bias_->t.data, ch.row0, ch.count, ch.n,
                             (float*)cp.data, (float*)cl.data, out.data, 2, (int)width_, c.stream);
        } else {
            K::linear_scan((const float*)a.data, (const float*)g.data, yx.data, dtype, 2 * width_, (const float*)y_bias_->t.data, state + conv_part, row,
                           c.dev.cu, c.dev.seq_new, c.dev.seq_slot, out.data, c.n_seqs, (int)width_, c.stream);
        }
        if (stream) {
            add_product(c, *stream, out, w_o_);
            return Tensor();
        }
        return linear(c, out, w_o_, nullptr, dtype).t;
    }

private:
    static const int SCAN_CHUNK = 32;
    int64_t hidden_, width_;
    int blocks_, taps_;
    double decay_scale_;
    std::string n_y_, n_yb_, n_x_, n_xb_, n_conv_, n_convb_, n_a_, n_ab_, n_i_, n_ib_, n_decay_, n_o_;
    Weight w_yx_, w_o_;
    OwnedPtr y_bias_, x_bias_, conv_w_, conv_b_, gate_a_, gate_i_, gate_a_b_, gate_i_b_, decay_c_;
    Loaded stored_;
};

// ---- mamba2 --------------------------------------------------------------------------------------------
// params: hidden, heads, head_dim (a head's values), state (rows of a head's state), groups (heads that share B and C), conv (taps),
// norm_groups, eps; names {in, conv, conv_bias, dt_bias, a_log, d, norm, o}.
class Mamba2 : public Mixer {
public:
    Mamba2(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "mamba2", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        heads_ = (int)r.integer("heads", 1);
        p_dim_ = (int)r.integer("head_dim", 1);
        n_state_ = (int)r.integer("state", 1);
        groups_ = (int)r.integer("groups", 1);
        taps_ = (int)r.integer("conv", 1);
        norm_groups_ = (int)r.integer("norm_groups", 1);
        eps_ = (float)r.number("eps");
        inner_ = (int64_t)heads_ * p_dim_;
        conv_ch_ = inner_ + 2LL * groups_ * n_state_;
        total_ = 2 * inner_ + 2LL * groups_ * n_state_ + heads_;
        if (heads_ % groups_) raise(TQE_ERR_CONFIG, "mamba2: %d heads do not fall into %d groups", heads_, groups_);
        if (inner_ % norm_groups_) raise(TQE_ERR_CONFIG, "mamba2: %lld values do not fall into %d parts of the norm", (long long)inner_, norm_groups_);
        if (taps_ > K::conv_max_taps.raw()) raise(TQE_ERR_CONFIG, "mamba2: a convolution of %d taps is more than the kernels take (%d)", taps_, K::conv_max_taps.raw());
        if (n_state_ > K::ssm_max_state.raw()) raise(TQE_ERR_CONFIG, "mamba2: a state of %d rows is more than the kernels take (%d)", n_state_, K::ssm_max_state.raw());
        const Json& n = spec.params["names"];
        n_in_ = name_of(n, "in", "in_proj.weight"); n_conv_ = name_of(n, "conv", "conv1d.weight"); n_convb_ = name_of(n, "conv_bias", "conv1d.bias");
        n_dtb_ = name_of(n, "dt_bias", "dt_bias"); n_alog_ = name_of(n, "a_log", "A_log"); n_d_ = name_of(n, "d", "D"); n_norm_ = name_of(n, "norm", "norm.weight");
        n_o_ = name_of(n, "o", "out_proj.weight");
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        TensorSpec conv = matrix(conv_ch_, taps_); conv.std_dev = 0.3;
        TensorSpec norm = vector_of(inner_, 0.1); norm.init = "one_plus_normal";
        return {{n_in_, matrix(total_, hidden_)}, {n_conv_, conv}, {n_convb_, vector_of(conv_ch_, 0.1)}, {n_dtb_, vector_of(heads_, 0.5)},
                {n_alog_, vector_of(heads_, 0.5)}, {n_d_, vector_of(heads_, 0.5)}, {n_norm_, norm}, {n_o_, matrix(hidden_, inner_)}};
    }
    void load(Loaded& t, hipStream_t stream) override {
        // (rows up to a multiple of 16, so that the product's rows stay at multiples of 16 bytes whatever the sizes)
        OwnedPtr in = stack_rows({take(t, n_in_)}, stream, 16);
        row_ = in->t.shape[0];
        w_in_ = make_weight(in, 1, false, stream);
        w_o_ = make_weight(take(t, n_o_), 1, false, stream);
        conv_w_ = as_floats(take(t, n_conv_), stream);
        conv_b_ = as_floats(take(t, n_convb_), stream);
        dt_bias_ = as_floats(take(t, n_dtb_), stream);
        a_log_ = as_floats(take(t, n_alog_), stream);
        d_ = as_floats(take(t, n_d_), stream);
        norm_w_ = as_floats(take(t, n_norm_), stream);
        stored_ = t;
        for (const std::string& big : {n_in_, n_o_}) stored_.erase(big);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "in.weight") return w_in_.rows;
        if (name == "o.weight") return w_o_.rows;
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    const char* trace_name() const override { return "mamba2"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({(total_ + 15) / 16 * 16, hidden_});
        out.push_back({hidden_, inner_});
    }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::State;
        n.state_shape = {(int64_t)(taps_ - 1) * conv_ch_ + (int64_t)heads_ * n_state_ * p_dim_};
        n.state_dtype = F32;
        return n;
    }
    bool adds_to_stream(const StepContext& c) const override { return fusable(c.n_tokens, w_o_, true) || leaves_sums(c.n_tokens, w_o_); }
    bool folds_norm(const StepContext& c) const override { return fusable(c.n_tokens, w_in_); }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (entry.kind != CacheNeed::State || !entry.writes) raise(TQE_ERR_STATE, "mamba2 was given no state of its own in the cache");
        if (last_rows) raise(TQE_ERR_STATE, "mamba2 takes all rows of the step");
        const int64_t n = x.rows();
        const int dtype = x.lazy ? BF16 : x.x.dtype;
        const long long row = entry.state.cols(), conv_part = (long long)(taps_ - 1) * conv_ch_;
        float* state = (float*)entry.state.data + entry.state_offset;
        const Tensor zxbcdt = x.lazy ? linear_of_norm(c, x.norm, w_in_, dtype) : linear(c, x.x, w_in_, nullptr, dtype).t;          // [z | x | B | C | dt | padding]
        Tensor xbc = c.alloc(F32, {n, conv_ch_}), y = c.alloc(F32, {n, inner_});
        if (c.all_decode) {
            K::conv_state_step(at(zxbcdt, inner_), dtype, row_, nullptr, (const float*)conv_w_->t.data, (const float*)conv_b_->t.data, taps_, 1, state, row,
                               c.dev.tok_seq, c.dev.seq_slot, (float*)xbc.data, (int)n, (int)conv_ch_, c.stream);
        } else {
            K::conv_state(at(zxbcdt, inner_), dtype, row_, nullptr, (const float*)conv_w_->t.data, (const float*)conv_b_->t.data, taps_, 1, state, row,
                          c.dev.tok_seq, c.dev.tok_pos, c.dev.seq_slot, c.dev.seq_start, (float*)xbc.data, (int)n, (int)conv_ch_, c.stream);
            K::conv_state_update(at(zxbcdt, inner_), dtype, row_, nullptr, taps_, state, row, c.dev.cu, c.dev.seq_new, c.dev.seq_slot, c.n_seqs, (int)conv_ch_,
                                 c.stream);
        }
        if (in_chunks(c, dtype)) {
            const Chunks ch = c.chunks(SCAN_CHUNK);
            const int64_t per_head = (int64_t)n_state_ * p_dim_;
            Tensor dt = c.alloc(F32, {n, heads_}), decay = c.alloc(F32, {n, heads_});
            Tensor cs = c.alloc(F32, {ch.n, heads_, per_head}), cd = c.alloc(F32, {ch.n, heads_});
            K::ssm_steps(at(zxbcdt, inner_ + conv_ch_), dtype, row_, (const float*)dt_bias_->t.data, (const float*)a_log_->t.data, (float*)dt.data,
                         (float*)decay.data, (int)n, heads_, c.stream);
            K::ssm_chunks((const float*)xbc.data, conv_ch_, (const float*)dt.data, (const float*)decay.data, (const float*)d_->t.data, ch.row0, ch.count, ch.n,
                          (float*)cs.data, (float*)cd.data, nullptr, 1, heads_, groups_, n_state_, p_dim_, c.stream);
            K::chunk_carry((const float*)cd.data, heads_, (int)per_head, (float*)cs.data, ch.seq_first, c.dev.seq_slot, state + conv_part, row, c.n_seqs,
                           heads_ * per_head, c.stream);
            K::ssm_chunks((const float*)xbc.data, conv_ch_, (const float*)dt.data, (const float*)decay.data, (const float*)d_->t.data, ch.row0, ch.count, ch.n,
                          (float*)cs.data, (float*)cd.data, (float*)y.data, 2, heads_, groups_, n_state_, p_dim_, c.stream);
        } else {
            K::ssm_scan((const float*)xbc.data, conv_ch_, at(zxbcdt, inner_ + conv_ch_), dtype, row_, (const float*)dt_bias_->t.data, (const float*)a_log_->t.data,
                        (const float*)d_->t.data, state + conv_part, row, c.dev.cu, c.dev.seq_new, c.dev.seq_slot, (float*)y.data, c.n_seqs, heads_, groups_,
                        n_state_, p_dim_, c.stream);
        }
        Tensor out = c.alloc(dtype, {n, inner_});
        K::gated_part_norm((const float*)y.data, zxbcdt.data, dtype, row_, (const float*)norm_w_->t.data, eps_, out.data, (int)n, (int)inner_, norm_groups_,
                           c.stream);
        if (stream) {
            add_product(c, *stream, out, w_o_);
            return Tensor();
        }
        return linear(c, out, w_o_, nullptr, dtype).t;
    }

private:
    static const int SCAN_CHUNK = 64;
    int64_t hidden_, inner_, conv_ch_, total_, row_ = 0;
    int heads_, p_dim_, n_state_, groups_, taps_, norm_groups_;
    float eps_;
    std::string n_in_, n_conv_, n_convb_, n_dtb_, n_alog_, n_d_, n_norm_, n_o_;
    Weight w_in_, w_o_;
    OwnedPtr conv_w_, conv_b_, dt_bias_, a_log_, d_, norm_w_;
    Loaded stored_;
};

}  // namespace

void register_recurrent_parts() {
    register_kind("mixer", "rglru", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<RGLRU>(s, e); });
    register_kind("mixer", "mamba2", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<Mamba2>(s, e); });
}

}  // namespace tq
