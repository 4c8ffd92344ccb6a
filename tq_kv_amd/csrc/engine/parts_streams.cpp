// A layer norm with weight and bias, and a block that keeps the residual stream in several copies.
//
//   norm  layer_norm   (x - mean) / sqrt(var + eps) w + b, the variance the mean of the squared deviations; float32 arithmetic.
//                      params: size, eps; optional tensor (the weight's name, "weight" unless given; may be empty) and bias_tensor
//                      ("bias" unless given).
//   block multi_stream pre-norm around a mixer and an optional feed-forward, with `streams` copies X[0..S) of the stream in place of
//                      the one.  A sublayer reads u = sum_s in[s] X[s], computes y = part(norm(u)), and all copies are updated at
//                      once from the old ones: X'[r] = sum_s mix[s, r] X[s] + out[r] y.  Every copy starts as the stream the block
//                      is given (the embedding's output); the last block of a model leaves the copies' sum in the stream.  Without
//                      `streams` there is one copy with in = mix = out = 1: the plain pre-norm block x' = x + part(norm(x)).
//                      token_shift: what the mixer reads is n_t + (n_(t-1) - n_t) mu with n = norm(u) and a learned mu per channel;
//                      the last n of a sequence is kept in the cache's state row, behind the mixer's own state.
//                      params: hidden, mixer, feed_forward (or null), mixer_norm, ff_norm (norm part specs), streams (or null),
//                      token_shift; names {mixer, feed_forward, mixer_norm, ff_norm, mixer_streams, ff_streams, shift}: prefixes of the
//                      parts' tensors and the names of the block's own: <mixer_streams>.in [S], .out [S], .mix [S, S], shift [hidden].
//
// The update of the copies that a sublayer's output brings is not run on its own: it rides with the next reading of the copies (one
// pass over them per sublayer), across blocks too, as the stream's pending update.
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

// a loaded tensor as float32 on the device
OwnedPtr as_floats(const OwnedPtr& p, hipStream_t stream) {
    if (p->t.dtype == F32) return p;
    std::vector<int64_t> dims(p->t.shape, p->t.shape + p->t.ndim);
    OwnedPtr out = make_owned(F32, dims);
    if (!null_device()) K::convert(p->t.data, p->t.dtype, out->t.data, F32, (long long)p->t.numel(), stream);
    stream_synchronize(stream);
    return out;
}

OwnedPtr constant_floats(const std::vector<float>& v) {
    OwnedPtr p = make_owned(F32, {(int64_t)v.size()});
    copy_to_device(p->t.data, v.data(), v.size() * 4, nullptr);
    stream_synchronize(nullptr);
    return p;
}

class LayerNorm : public Norm {
public:
    LayerNorm(const PartSpec& spec, BuildEnv& env) : act_dtype_(env.act_dtype) {
        KeyReader r(spec.params, "layer_norm", TQE_ERR_ARGUMENT);
        size_ = r.integer("size", 1);
        eps_ = (float)r.number("eps");
        n_w_ = r.string_or("tensor", "weight");
        n_b_ = r.string_or("bias_tensor", "bias");
        if (n_w_ == n_b_) raise(TQE_ERR_ARGUMENT, "layer_norm: weight and bias under one name '%s'", n_w_.c_str());
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        TensorSpec w; w.shape = {size_}; w.init = "one_plus_normal"; w.std_dev = 0.1;
        TensorSpec b; b.shape = {size_}; b.std_dev = 0.1;
        return {{n_w_, w}, {n_b_, b}};
    }
    void load(Loaded& t, hipStream_t stream) override {
        stored_ = t;
        w_ = as_floats(take(t, n_w_), stream);
        b_ = as_floats(take(t, n_b_), stream);
    }
    OwnedPtr held(const std::string& name) const override {
        auto it = stored_.find(name);
        return it == stored_.end() ? nullptr : it->second;
    }
    const char* trace_name() const override { return "rms-norm"; }
    int64_t size() const override { return size_; }
    const float* weight() const { return (const float*)w_->t.data; }
    const float* bias() const { return (const float*)b_->t.data; }
    float eps() const { return eps_; }

    void forward(StepContext& c, const Tensor& x, Tensor& out) override {
        K::add_layer_norm(nullptr, x.data, x.dtype, nullptr, (int)x.shape[0], weight(), bias(), eps_, out.data, out.dtype, (int)size_, 0, c.stream);
    }
    void add_norm(StepContext& c, Tensor& h, const Pending& delta, Tensor& out) override {
        if (delta.kind == Pending::Sums) raise(TQE_ERR_STATE, "layer_norm takes no unfinished product");
        const bool d = delta.kind == Pending::Plain;
        K::add_layer_norm((float*)h.data, d ? delta.t.data : nullptr, d ? delta.t.dtype : 0, nullptr, (int)h.shape[0], weight(), bias(), eps_, out.data, out.dtype,
                          (int)size_, d ? 1 : 0, c.stream);
    }
    void gather_add_norm(StepContext& c, const Tensor& h, const Pending& delta, const int32_t* rows, int64_t n_rows, Tensor& out) override {
        if (delta.kind == Pending::Sums) raise(TQE_ERR_STATE, "layer_norm takes no unfinished product");
        const bool d = delta.kind == Pending::Plain;
        K::add_layer_norm((float*)h.data, d ? delta.t.data : nullptr, d ? delta.t.dtype : 0, rows, (int)n_rows, weight(), bias(), eps_, out.data, out.dtype,
                          (int)size_, 0, c.stream);
    }

private:
    int act_dtype_;
    int64_t size_;
    float eps_;
    std::string n_w_, n_b_;
    OwnedPtr w_, b_;
    Loaded stored_;
};

class MultiStreamBlock : public Block {
public:
    MultiStreamBlock(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "multi_stream block", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        has_streams_ = r.has("streams");
        streams_ = has_streams_ ? (int)r.integer("streams", 1) : 1;
        shift_ = r.boolean_or("token_shift", false);
        if (streams_ > K::streams_max.raw()) raise(TQE_ERR_CONFIG, "multi_stream block: %d copies of the stream are more than the kernels take (%d)", streams_, K::streams_max.raw());
        const Json& names = spec.params["names"];
        auto name = [&](const char* role, const char* fallback) { return names[role].is_string() ? names[role].as_string() : std::string(fallback); };
        auto one = [&](const char* role, const char* category, bool optional) -> std::shared_ptr<Part> {
            const Json& p = spec.params[role];
            if (p.is_null()) {
                if (optional) return nullptr;
                raise(TQE_ERR_ARGUMENT, "multi_stream block: no '%s' given", role);
            }
            std::shared_ptr<Part> part = build_part(category, PartSpec::from_json(p, role), env);
            if (!names[role].is_string()) raise(TQE_ERR_ARGUMENT, "multi_stream block: no tensor-name prefix for '%s'", role);
            roles_.push_back({role, names[role].as_string(), part});
            return part;
        };
        mixer_ = std::dynamic_pointer_cast<Mixer>(one("mixer", "mixer", false));
        feed_forward_ = std::dynamic_pointer_cast<FeedForward>(one("feed_forward", "feed_forward", true));
        mixer_norm_ = std::dynamic_pointer_cast<Norm>(one("mixer_norm", "norm", false));
        if (feed_forward_) ff_norm_ = std::dynamic_pointer_cast<Norm>(one("ff_norm", "norm", false));
        if (!mixer_ || !mixer_norm_ || (feed_forward_ && !ff_norm_)) raise(TQE_ERR_ARGUMENT, "multi_stream block: a part is of the wrong category");
        n_hc_[0] = name("mixer_streams", "mixer_streams");
        n_hc_[1] = name("ff_streams", "ff_streams");
        n_shift_ = name("shift", "shift");
        const CacheNeed inner = mixer_->cache_need();
        if (inner.kind != CacheNeed::None && inner.has_state() && inner.state_dtype != F32)
            raise(TQE_ERR_ARGUMENT, "multi_stream block: the mixer's state is not float32, the kept token's is");
        inner_state_ = 1;
        for (int64_t v : inner.state_shape) inner_state_ *= v;
        if (!inner.has_state()) inner_state_ = 0;
        graph_safe = true;
        for (const Role& role : roles_) graph_safe = graph_safe && role.part->graph_safe;
    }

    TensorSpecs tensors() const override {
        TensorSpecs out;
        for (const Role& r : roles_)
            for (const auto& t : r.part->tensors()) out.push_back({r.prefix + t.first, t.second});
        if (has_streams_)
            for (int q = 0; q < (feed_forward_ ? 2 : 1); ++q) {
                // weights near the plain residual sum: every copy read and written with about 1 / S and 1, mixed with about the identity
                TensorSpec in; in.shape = {streams_}; in.init = "one_plus_normal"; in.std_dev = 0.1;
                TensorSpec outw = in;
                TensorSpec mix; mix.shape = {streams_, streams_}; mix.std_dev = 0.3;
                out.push_back({n_hc_[q] + ".in", in});
                out.push_back({n_hc_[q] + ".out", outw});
                out.push_back({n_hc_[q] + ".mix", mix});
            }
        if (shift_) { TensorSpec mu; mu.shape = {hidden_}; mu.std_dev = 0.3; out.push_back({n_shift_, mu}); }
        return out;
    }
    void load(Loaded& tensors, hipStream_t stream) override {
        for (const Role& r : roles_) {
            Loaded own;
            for (const auto& t : r.part->tensors()) own[t.first] = take(tensors, r.prefix + t.first);
            r.part->load(own, stream);
        }
        for (int q = 0; q < (feed_forward_ ? 2 : 1); ++q) {
            if (has_streams_) {
                in_[q] = as_floats(take(tensors, n_hc_[q] + ".in"), stream);
                out_[q] = as_floats(take(tensors, n_hc_[q] + ".out"), stream);
                mix_[q] = as_floats(take(tensors, n_hc_[q] + ".mix"), stream);
            } else {
                in_[q] = out_[q] = mix_[q] = constant_floats({1.f});
            }
        }
        ones_ = constant_floats(std::vector<float>((size_t)streams_, 1.f));
        if (shift_) mu_ = as_floats(take(tensors, n_shift_), stream);
        own_ = tensors;
    }
    OwnedPtr held(const std::string& name) const override {
        for (const Role& r : roles_)
            if (name.compare(0, r.prefix.size(), r.prefix) == 0)
                if (OwnedPtr p = r.part->held(name.substr(r.prefix.size()))) return p;
        auto it = own_.find(name);
        return it == own_.end() ? nullptr : it->second;
    }
    Json describe() const override {
        Json j = Part::describe();
        Json parts = Json::object();
        for (const Role& r : roles_) parts.set(r.role, r.part->describe());
        j.set("parts", parts);
        return j;
    }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        for (const Role& r : roles_) r.part->product_shapes(out);
    }
    // the mixer's need, and behind its state the row of the kept token
    CacheNeed cache_need() const override {
        CacheNeed n = mixer_->cache_need();
        if (!shift_) return n;
        if (n.kind == CacheNeed::None) n.kind = CacheNeed::State;
        n.state_shape = {inner_state_ + hidden_};
        n.state_dtype = F32;
        return n;
    }
    Norm* first_norm() override { return nullptr; }        // the norm in front of the mixer runs inside the block's own kernel
    Mixer* mixer() override { return mixer_.get(); }

    Stream* forward(StepContext& c, Stream* stream, const CacheEntry& entry, Norm*, bool last) override {
        const int64_t n = stream->h.shape[0];
        const int S = streams_;
        if (stream->h.shape[1] != hidden_) raise(TQE_ERR_STATE, "multi_stream block: a stream of %lld values, the block was built for %lld", (long long)stream->h.shape[1], (long long)hidden_);
        if (!stream->copies.defined()) {
            if (stream->pending.kind != Pending::Nothing) raise(TQE_ERR_STATE, "multi_stream block: the stream it is given has an update that was not added");
            stream->copies = Tensor(c.ws->alloc_for_step((size_t)(n * S * hidden_) * 4), F32, {n, S, hidden_});
            K::streams_fill((const float*)stream->h.data, (float*)stream->copies.data, S, (int)n, (int)hidden_, c.stream);
            stream->invalidate();
        } else if (stream->copies.shape[1] != S) {
            raise(TQE_ERR_STATE, "multi_stream block: the stream comes in %lld copies, the block keeps %d", (long long)stream->copies.shape[1], S);
        }
        if (stream->pending.kind == Pending::Sums) raise(TQE_ERR_STATE, "multi_stream block: the block before left an unfinished product on the stream");
        // the mixer
        Activation x;
        x.x = read(c, *stream, 0, shift_ ? F32 : c.act_dtype);
        if (shift_) {
            if (!entry.state.defined()) raise(TQE_ERR_STATE, "multi_stream block: no state row in the cache for the kept token");
            float* state = (float*)entry.state.data + entry.state_offset + inner_state_;
            Tensor shifted = c.alloc(c.act_dtype, {n, hidden_});
            K::token_shift((const float*)x.x.data, (const float*)mu_->t.data, state, entry.state.cols(), c.dev.tok_seq, c.dev.tok_pos, c.dev.seq_start, c.dev.seq_slot,
                           shifted.data, shifted.dtype, (int)n, (int)hidden_, c.all_decode ? 1 : 0, c.stream);
            if (!c.all_decode)
                K::shift_remember((const float*)x.x.data, state, entry.state.cols(), c.dev.cu, c.dev.seq_new, c.dev.seq_slot, c.n_seqs, (int)hidden_, c.stream);
            x.x = shifted;
        }
        Tensor y;
        {
            Span span(mixer_->trace_name());
            y = mixer_->forward(c, x, entry, nullptr, false);
        }
        leave(*stream, y, 0);
        if (feed_forward_) {
            x.x = read(c, *stream, 1, c.act_dtype);
            {
                Span span(feed_forward_->trace_name());
                y = feed_forward_->forward(c, x, nullptr);
            }
            leave(*stream, y, 1);
        }
        if (last) {
            // nothing but the head reads the stream after this block: the copies' sum, with the last update on its way
            K::streams_step((float*)stream->copies.data, S, stream->pending.t.data, stream->pending.t.dtype, stream->copies_mix, stream->copies_out,
                            (const float*)ones_->t.data, nullptr, nullptr, 0.f, (float*)stream->h.data, nullptr, 0, (int)n, (int)hidden_, wide(c), c.stream);
            stream->pending = Pending();
            stream->copies_mix = stream->copies_out = nullptr;
        }
        return stream;
    }

private:
    struct Role { std::string role, prefix; std::shared_ptr<Part> part; };

    // bfloat16 steps of few tokens give a row more threads; 32-bit steps keep one order of a row's sums whatever the step holds
    static int wide(const StepContext& c) { return c.act_dtype == BF16 && c.n_tokens <= 64 ? 1 : 0; }

    // what sublayer q reads: the pending update of the copies, then the norm of their weighted sum
    Tensor read(StepContext& c, Stream& s, int q, int dtype) {
        Norm* norm = q == 0 ? mixer_norm_.get() : ff_norm_.get();
        Span span(norm->trace_name());
        const int64_t n = s.h.shape[0];
        const bool pending = s.pending.kind == Pending::Plain;
        if (pending && (!s.copies_mix || !s.copies_out)) raise(TQE_ERR_STATE, "multi_stream block: an update of the stream without the copies' weights");
        Tensor out = c.alloc(dtype, {n, hidden_});
        const LayerNorm* ln = dynamic_cast<const LayerNorm*>(norm);
        if (ln) {
            K::streams_step((float*)s.copies.data, streams_, pending ? s.pending.t.data : nullptr, pending ? s.pending.t.dtype : 0, s.copies_mix, s.copies_out,
                            (const float*)in_[q]->t.data, ln->weight(), ln->bias(), ln->eps(), nullptr, out.data, out.dtype, (int)n, (int)hidden_, wide(c), c.stream);
        } else {
            // another norm: the weighted sum from the kernel, the norm as a step of its own
            Tensor u = c.alloc(F32, {n, hidden_});
            K::streams_step((float*)s.copies.data, streams_, pending ? s.pending.t.data : nullptr, pending ? s.pending.t.dtype : 0, s.copies_mix, s.copies_out,
                            (const float*)in_[q]->t.data, nullptr, nullptr, 0.f, (float*)u.data, nullptr, 0, (int)n, (int)hidden_, wide(c), c.stream);
            norm->forward(c, u, out);
        }
        s.pending = Pending();
        s.copies_mix = s.copies_out = nullptr;
        s.invalidate();
        return out;
    }
    void leave(Stream& s, const Tensor& y, int q) {
        if (y.shape[0] != s.h.shape[0] || y.cols() != hidden_)
            raise(TQE_ERR_STATE, "multi_stream block: a part returned %s for a stream of [%lld, %lld]", y.describe().c_str(), (long long)s.h.shape[0], (long long)hidden_);
        s.pending = Pending::of(y);
        s.copies_mix = (const float*)mix_[q]->t.data;
        s.copies_out = (const float*)out_[q]->t.data;
    }

    int64_t hidden_, inner_state_ = 0;
    int streams_ = 1;
    bool has_streams_ = false, shift_ = false;
    std::string n_hc_[2], n_shift_;
    std::vector<Role> roles_;
    std::shared_ptr<Mixer> mixer_;
    std::shared_ptr<FeedForward> feed_forward_;
    std::shared_ptr<Norm> mixer_norm_, ff_norm_;
    OwnedPtr in_[2], out_[2], mix_[2], ones_, mu_;
    Loaded own_;
};

}  // namespace

void register_streams_parts() {
    register_kind("norm", "layer_norm", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<LayerNorm>(s, e); });
    register_kind("block", "multi_stream", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<MultiStreamBlock>(s, e); });
}

}  // namespace tq
