// A feed-forward of routed experts.
//
// Each token goes through `top` of `n_experts` small gated feed-forwards.  The router's logits
// z = W_r x are computed in float32, s = softmax(z) runs over all experts, the `top` largest are
// chosen, and their outputs are added up with the weights s * router_scale (not renormalised).  An
// expert is down(gate(gate_proj x, up_proj x)) with the gate its params name (Gate in linear.h); it
// has no biases.  A shared expert (any feed-forward part, optional) runs for every token and is
// added.
//
// The step's (token, expert) pairs are grouped by expert on the device (moe.hip): the products run
// over tiles of rows that belong to one expert, from lists that stay on the device, so the
// launches are the same whatever the router chose and a step can be captured as a graph.
//
// Variants, all parameters: gated false makes an expert down(f(up_proj x)), f the gate's function of one product
// (relu2: max(z, 0)^2), without a gate product and its tensor; normalize "chosen" makes the weights the softmax over
// the chosen logits alone (times router_scale); shared_gate names a tensor [1, hidden] whose product with x, through
// a sigmoid, multiplies the shared expert's output token by token; score "sigmoid" makes an expert's score sigmoid(z) on its own
// instead of the softmax over all; weight_on "input" multiplies an expert's input by the weight (the output is then the plain sum of
// E(w x) over the chosen experts, which is not w E(x) since an expert is not linear).
//
// params: hidden, inter, n_experts, top, router_scale, gate / limit / alpha, gated, normalize, score, weight_on, shared (a feed-forward
// part spec, or null), shared_gate (a tensor's name, or null); optional names {router, expert (with %d for the expert's number), gate, up,
// down, shared}.  Tensors: router [experts, hidden]; per expert gate, up [inter, hidden], down
// [hidden, inter]; the shared expert's own under its prefix.
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

class RoutedExperts : public FeedForward {
public:
    RoutedExperts(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "routed_experts", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        inter_ = r.integer("inter", 1);
        n_experts_ = (int)r.integer("n_experts", 1);
        top_ = (int)r.integer("top", 1);
        router_scale_ = (float)r.number_or("router_scale", 1.0);
        gate_ = Gate::from_params(r, "routed_experts");
        gated_ = r.boolean_or("gated", true);
        const std::string normalize = r.string_or("normalize", "all");
        if (normalize != "all" && normalize != "chosen") raise(TQE_ERR_ARGUMENT, "routed_experts: unknown normalize '%s' (known: all, chosen)", normalize.c_str());
        renormalize_ = normalize == "chosen";
        const std::string score = r.string_or("score", "softmax");
        if (score != "softmax" && score != "sigmoid") raise(TQE_ERR_ARGUMENT, "routed_experts: unknown score '%s' (known: sigmoid, softmax)", score.c_str());
        sigmoid_scores_ = score == "sigmoid";
        const std::string weight_on = r.string_or("weight_on", "output");
        if (weight_on != "output" && weight_on != "input") raise(TQE_ERR_ARGUMENT, "routed_experts: unknown weight_on '%s' (known: input, output)", weight_on.c_str());
        weight_on_input_ = weight_on == "input";
        n_shared_gate_ = r.string_or("shared_gate", "");
        if (top_ > n_experts_) raise(TQE_ERR_ARGUMENT, "routed_experts: top %d of %d experts", top_, n_experts_);
        const int most = K::moe_max_experts.raw();
        if (n_experts_ > most) raise(TQE_ERR_CONFIG, "routed_experts: %d experts are more than the kernels take (%d)", n_experts_, most);
        const Json& names = spec.params["names"];
        auto name = [&](const char* role, const char* fallback) { return names[role].is_string() ? names[role].as_string() : std::string(fallback); };
        n_router_ = name("router", "router");
        n_expert_ = name("expert", "e%d.");
        n_gate_ = name("gate", "gate");
        n_up_ = name("up", "up");
        n_down_ = name("down", "down");
        n_shared_ = name("shared", "shared.");
        if (n_expert_.find("%d") == std::string::npos || n_expert_.find('%') != n_expert_.rfind('%'))
            raise(TQE_ERR_ARGUMENT, "routed_experts: the experts' prefix '%s' must hold one %%d", n_expert_.c_str());
        graph_safe = true;
        if (!spec.params["shared"].is_null()) {
            shared_ = std::dynamic_pointer_cast<FeedForward>(build_part("feed_forward", PartSpec::from_json(spec.params["shared"], "routed_experts: shared"), env));
            if (!shared_) raise(TQE_ERR_ARGUMENT, "routed_experts: the shared expert is no feed-forward");
            graph_safe = shared_->graph_safe;
        }
        if (!n_shared_gate_.empty() && !shared_) raise(TQE_ERR_ARGUMENT, "routed_experts: a gate for a shared expert that is not there");
    }

    std::string expert_prefix(int e) const {
        std::string s = n_expert_;
        s.replace(s.find("%d"), 2, std::to_string(e));
        return s;
    }
    TensorSpecs tensors() const override {
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        TensorSpecs t = {{n_router_, w(n_experts_, hidden_)}};
        for (int e = 0; e < n_experts_; ++e) {
            const std::string p = expert_prefix(e);
            if (gated_) t.push_back({p + n_gate_, w(inter_, hidden_)});
            t.push_back({p + n_up_, w(inter_, hidden_)});
            t.push_back({p + n_down_, w(hidden_, inter_)});
        }
        if (shared_)
            for (const auto& s : shared_->tensors()) t.push_back({n_shared_ + s.first, s.second});
        if (!n_shared_gate_.empty()) t.push_back({n_shared_gate_, w(1, hidden_)});
        return t;
    }
    void load(Loaded& t, hipStream_t stream) override {
        router_ = take(t, n_router_);
        // all experts' weights in two tensors: [experts, gate rows then up rows, hidden] and [experts, hidden, inter]
        std::vector<OwnedPtr> gu, down;
        for (int e = 0; e < n_experts_; ++e) {
            const std::string p = expert_prefix(e);
            if (gated_) gu.push_back(take(t, p + n_gate_));
            gu.push_back(take(t, p + n_up_));
            down.push_back(take(t, p + n_down_));
        }
        gate_up_ = stack_rows(gu, stream);
        down_ = stack_rows(down, stream);
        if (shared_) {
            Loaded own;
            for (const auto& s : shared_->tensors()) own[s.first] = take(t, n_shared_ + s.first);
            shared_->load(own, stream);
        }
        if (!n_shared_gate_.empty()) shared_gate_ = take(t, n_shared_gate_);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == n_router_) return router_;
        if (!n_shared_gate_.empty() && name == n_shared_gate_) return shared_gate_;
        if (name == "experts.gate_up") return gate_up_;
        if (name == "experts.down") return down_;
        if (shared_ && name.compare(0, n_shared_.size(), n_shared_) == 0) return shared_->held(name.substr(n_shared_.size()));
        return nullptr;
    }
    const char* trace_name() const override { return "attn-mlp"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        if (shared_) shared_->product_shapes(out);
    }

    Tensor forward(StepContext& c, const Activation& x, Stream*) override {
        if (x.lazy) raise(TQE_ERR_STATE, "routed_experts takes no folded norm");
        const int64_t n = x.x.shape[0];
        const int dtype = x.x.dtype;
        const int64_t pairs = n * top_;
        // bfloat16 on the matrix cores, in tiles whose size follows the rows an expert gets on average; else the plain kernel
        const bool on_cores = dtype == BF16 && gate_up_->t.dtype == BF16 && down_->t.dtype == BF16 && policy().skinny && hidden_ % 8 == 0 &&
                              inter_ % 8 == 0 && K::grouped_supported.raw((int)hidden_) != 0;
        const int64_t per_expert = pairs / n_experts_;
        const int tile_m = !on_cores ? K::moe_tile_rows.raw() : per_expert >= 48 ? 64 : per_expert >= 24 ? 32 : 16;
        const int max_tiles = K::moe_max_tiles.raw((int)pairs, n_experts_, tile_m);
        Tensor idx = c.alloc(I32, {n, top_}), weight = c.alloc(F32, {n, top_});
        Tensor pair_pos = c.alloc(I32, {pairs}), sorted_tok = c.alloc(I32, {pairs});
        Tensor tiles = c.alloc(I32, {3, max_tiles}), n_tiles = c.alloc(I32, {4});
        int32_t* tile_expert = (int32_t*)tiles.data;
        int32_t* tile_row0 = tile_expert + max_tiles;
        int32_t* tile_rows = tile_row0 + max_tiles;
        // the shared expert's gate rides along with the router where both weights are of one type
        Tensor shared_scale;
        const bool gate_in_route = shared_gate_ && shared_gate_->t.dtype == router_->t.dtype;
        if (shared_gate_) shared_scale = c.alloc(F32, {n});
        K::moe_route(x.x.data, dtype, router_->t.data, router_->t.dtype, n_experts_, (int)hidden_, top_, router_scale_, (renormalize_ ? 1 : 0) | (sigmoid_scores_ ? 2 : 0), (int32_t*)idx.data,
                     (float*)weight.data, gate_in_route ? shared_gate_->t.data : nullptr, gate_in_route ? (float*)shared_scale.data : nullptr, (int)n, c.stream);
        K::moe_group((const int32_t*)idx.data, (int)n, top_, n_experts_, tile_m, (int32_t*)pair_pos.data, (int32_t*)sorted_tok.data, tile_expert, tile_row0,
                     tile_rows, (int32_t*)n_tiles.data, c.stream);
        Tensor shared_out;
        if (shared_) shared_out = shared_->forward(c, x, nullptr);
        if (shared_gate_ && !gate_in_route) {
            K::row_gate(x.x.data, dtype, shared_gate_->t.data, shared_gate_->t.dtype, (float*)shared_scale.data, (int)n, (int)hidden_, c.stream);
        }
        // an expert's first product: gate and up side by side, or up alone with the gate's function of it
        const int first = gated_ ? 1 : 2;
        const long long first_stride = (long long)(gated_ ? 2 : 1) * inter_ * hidden_;
        Tensor act = c.alloc(dtype, {pairs, inter_});
        Tensor y = c.alloc(dtype, {pairs, hidden_});
        // the weight on the experts' inputs: every pair's row is its token's times the pair's weight, and the sum below is a plain one
        const void* first_in = x.x.data;
        const int32_t* first_rows = (const int32_t*)sorted_tok.data;
        const float* sum_weight = (const float*)weight.data;
        if (weight_on_input_) {
            Tensor scaled = c.alloc(dtype, {pairs, hidden_}), unit = c.alloc(F32, {n, top_});
            K::moe_scale_rows(x.x.data, dtype, (const int32_t*)pair_pos.data, (const float*)weight.data, top_, scaled.data, (float*)unit.data, (int)n, (int)hidden_,
                              c.stream);
            first_in = scaled.data;
            first_rows = nullptr;
            sum_weight = (const float*)unit.data;
        }
        if (on_cores) {
            K::moe_product_mfma(first_in, first_rows, gate_up_->t.data, first_stride, act.data, (int)inter_,
                                (int)hidden_, first, gate_.kind, gate_.limit, gate_.alpha, tile_expert, tile_row0, tile_rows,
                                (const int32_t*)n_tiles.data, max_tiles, tile_m, c.stream);
            K::moe_product_mfma(act.data, nullptr, down_->t.data, (long long)(hidden_ * inter_), y.data, (int)hidden_, (int)inter_, 0, 0, 0.f, 1.f,
                                tile_expert, tile_row0, tile_rows, (const int32_t*)n_tiles.data, max_tiles, tile_m, c.stream);
        } else {
            K::moe_product(first_in, dtype, first_rows, gate_up_->t.data, gate_up_->t.dtype, first_stride,
                           act.data, (int)inter_, (int)hidden_, first, gate_.kind, gate_.limit, gate_.alpha, tile_expert, tile_row0, tile_rows,
                           (const int32_t*)n_tiles.data, max_tiles, c.stream);
            K::moe_product(act.data, dtype, nullptr, down_->t.data, down_->t.dtype, (long long)(hidden_ * inter_), y.data, (int)hidden_, (int)inter_, 0,
                           0, 0.f, 1.f, tile_expert, tile_row0, tile_rows, (const int32_t*)n_tiles.data, max_tiles, c.stream);
        }
        Tensor out = c.alloc(dtype, {n, hidden_});
        K::moe_combine(y.data, dtype, (const int32_t*)pair_pos.data, sum_weight, top_, shared_out.data,
                       shared_gate_ ? (const float*)shared_scale.data : nullptr, out.data, (int)n,
                       (int)hidden_, c.stream);
        return out;
    }

private:
    int64_t hidden_, inter_;
    int n_experts_, top_;
    float router_scale_;
    Gate gate_;
    bool gated_ = true, renormalize_ = false, sigmoid_scores_ = false, weight_on_input_ = false;
    std::string n_shared_gate_;
    OwnedPtr shared_gate_;
    std::string n_router_, n_expert_, n_gate_, n_up_, n_down_, n_shared_;
    std::shared_ptr<FeedForward> shared_;
    OwnedPtr router_, gate_up_, down_;
};

}  // namespace

void register_moe_parts() {
    register_kind("feed_forward", "routed_experts", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<RoutedExperts>(s, e); });
}

}  // namespace tq
