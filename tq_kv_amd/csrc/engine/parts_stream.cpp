// Parts around the residual stream that are no pre-norm arrangement:
//
//   block "output_norm"           x <- x + norm1(mixer(x)); x <- x + norm2(ff(x)): the parts read the stream itself and
//                                 only their outputs are normed.  The sum stays float32; the kernel that adds a normed
//                                 output also writes the stream in the activation type, which is what the next part reads.
//   position "pair_hash"          acts on the stream after the gather: adds the row (a * previous + b * token) mod n of a
//                                 table of n + 1 rows (the last row for a sequence's first token).  The previous token is
//                                 kept per sequence as a state of the cache, so a sequence may come in pieces.
//   feed_forward "activated"      down(f(up x)) with f a gate's function of one product (relu2: max(z, 0)^2).
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

// ---- hashed pairs ------------------------------------------------------------------------------------
// params: hidden, vocab, buckets, mul_prev, mul_cur, max_positions; optional tensor (the table's name inside the part's prefix).
class PairHash : public Position {
public:
    PairHash(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "pair_hash", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        vocab_ = r.integer("vocab", 1);
        buckets_ = r.integer("buckets", 1);
        mul_prev_ = r.integer("mul_prev", 0);
        mul_cur_ = r.integer("mul_cur", 0);
        max_positions = r.integer_or("max_positions", (long long)1 << 30, 1);
        tensor_ = r.string_or("tensor", "table");
        if (buckets_ >= ((long long)1 << 31) || mul_prev_ >= ((long long)1 << 31) || mul_cur_ >= ((long long)1 << 31))
            raise(TQE_ERR_CONFIG, "pair_hash: buckets and multipliers must be below 2^31");
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        TensorSpec t;
        t.shape = {buckets_ + 1, hidden_};
        return {{tensor_, t}};
    }
    void load(Loaded& t, hipStream_t) override { table_ = take(t, tensor_); }
    OwnedPtr held(const std::string& name) const override { return name == tensor_ ? table_ : nullptr; }
    bool acts_on_stream() const override { return true; }
    CacheNeed stream_state_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::State;
        n.state_shape = {1};
        n.state_dtype = I32;
        return n;
    }
    void add_to_stream(StepContext&, Tensor&) override { raise(TQE_ERR_STATE, "pair_hash needs its state: the previous token of every sequence"); }
    void add_to_stream_with(StepContext& c, Tensor& h, const CacheEntry& state) override { add(c, h, state, nullptr); }
    // the same, and the stream's rows in the activation type where that is bfloat16 (what the first part of a layer reads)
    void add_to_stream_copy(StepContext& c, Tensor& h, const CacheEntry& state, Tensor& copy) override { add(c, h, state, copy.dtype == BF16 ? copy.data : nullptr); }
    bool writes_stream_copy() const override { return true; }

private:
    void add(StepContext& c, Tensor& h, const CacheEntry& state, void* copy) {
        if (state.kind != CacheNeed::State || state.state.dtype != I32) raise(TQE_ERR_STATE, "pair_hash was given no state of the cache");
        int32_t* last = (int32_t*)state.state.data;
        K::pair_embed(table_->t.data, table_->t.dtype, (int)buckets_, mul_prev_, mul_cur_, c.dev.tokens, c.dev.tok_seq, c.dev.tok_pos, c.dev.seq_slot,
                      c.dev.seq_start, last, (float*)h.data, c.n_tokens, (int)hidden_, (int)vocab_, copy, c.all_decode ? 1 : 0, c.stream);
        // otherwise its own launch: the first token of a sequence's piece reads what the last one writes
        if (!c.all_decode) K::remember_tokens(c.dev.tokens, c.dev.cu, c.dev.seq_new, c.dev.seq_slot, last, c.n_seqs, c.stream);
    }
    int64_t hidden_, vocab_, buckets_, mul_prev_, mul_cur_;
    std::string tensor_;
    OwnedPtr table_;
};

// ---- a feed-forward of one product and its activation ---------------------------------------------------
// params: hidden, inter, gate (the function's name) / limit / alpha; optional names {up, down}.
class Activated : public FeedForward {
public:
    Activated(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "activated", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        inter_ = r.integer("inter", 1);
        act_ = Gate::from_params(r, "activated");
        const Json& names = spec.params["names"];
        n_up_ = names["up"].is_string() ? names["up"].as_string() : "up_proj.weight";
        n_down_ = names["down"].is_string() ? names["down"].as_string() : "down_proj.weight";
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        return {{n_up_, w(inter_, hidden_)}, {n_down_, w(hidden_, inter_)}};
    }
    void load(Loaded& t, hipStream_t stream) override {
        w_up_ = make_weight(take(t, n_up_), 1, false, stream);
        w_down_ = make_weight(take(t, n_down_), 1, false, stream);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == n_up_) return w_up_.rows;
        if (name == n_down_) return w_down_.rows;
        return nullptr;
    }
    const char* trace_name() const override { return "attn-mlp"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({inter_, hidden_});
        out.push_back({hidden_, inter_});
    }
    Tensor forward(StepContext& c, const Activation& x, Stream*) override {
        if (x.lazy) raise(TQE_ERR_STATE, "activated takes no folded norm");
        Tensor u = linear(c, x.x, w_up_, nullptr, x.x.dtype).t;
        K::unary_act(u.data, u.data, u.dtype, (long long)u.numel(), act_.kind, act_.limit, act_.alpha, c.stream);
        return linear(c, u, w_down_, nullptr, x.x.dtype).t;
    }

private:
    int64_t hidden_, inter_;
    Gate act_;
    std::string n_up_, n_down_;
    Weight w_up_, w_down_;
};

// ---- the block ---------------------------------------------------------------------------------------------
// params: mixer, feed_forward (or null), mixer_out_norm, ff_out_norm (part specs of norms; null: the output is added as it is);
// names: part -> tensor-name prefix inside the layer.
class OutputNormBlock : public Block {
public:
    OutputNormBlock(const PartSpec& spec, BuildEnv& env) {
        const Json& names = spec.params["names"];
        auto one = [&](const char* role, const char* category, bool optional) -> std::shared_ptr<Part> {
            const Json& p = spec.params[role];
            if (p.is_null()) {
                if (optional) return nullptr;
                raise(TQE_ERR_ARGUMENT, "output_norm block: no '%s' given", role);
            }
            std::shared_ptr<Part> part = build_part(category, PartSpec::from_json(p, role), env);
            if (!names[role].is_string()) raise(TQE_ERR_ARGUMENT, "output_norm block: no tensor-name prefix for '%s'", role);
            roles_.push_back({role, names[role].as_string(), part});
            return part;
        };
        mixer_ = std::dynamic_pointer_cast<Mixer>(one("mixer", "mixer", false));
        const bool has_ff = !spec.params["feed_forward"].is_null();
        feed_forward_ = std::dynamic_pointer_cast<FeedForward>(one("feed_forward", "feed_forward", true));
        mixer_out_norm_ = std::dynamic_pointer_cast<Norm>(one("mixer_out_norm", "norm", true));
        ff_out_norm_ = has_ff ? std::dynamic_pointer_cast<Norm>(one("ff_out_norm", "norm", true)) : nullptr;
        if (!mixer_ || (has_ff && !feed_forward_)) raise(TQE_ERR_ARGUMENT, "output_norm block: a part is of the wrong category");
        graph_safe = true;
        for (const Role& r : roles_) graph_safe = graph_safe && r.part->graph_safe;
    }
    TensorSpecs tensors() const override {
        TensorSpecs out;
        for (const Role& r : roles_)
            for (const auto& t : r.part->tensors()) out.push_back({r.prefix + t.first, t.second});
        return out;
    }
    void load(Loaded& tensors, hipStream_t stream) override {
        for (const Role& r : roles_) {
            Loaded own;
            for (const auto& t : r.part->tensors()) own[t.first] = take(tensors, r.prefix + t.first);
            r.part->load(own, stream);
        }
    }
    OwnedPtr held(const std::string& name) const override {
        for (const Role& r : roles_)
            if (name.compare(0, r.prefix.size(), r.prefix) == 0)
                if (OwnedPtr p = r.part->held(name.substr(r.prefix.size()))) return p;
        return nullptr;
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
    CacheNeed cache_need() const override { return mixer_->cache_need(); }
    Norm* first_norm() override { return nullptr; }         // nothing norms the stream in front of this block
    Mixer* mixer() override { return mixer_.get(); }

    Stream* forward(StepContext& c, Stream* stream, const CacheEntry& entry, Norm*, bool last) override {
        const bool rows_only = last && c.prune_last && policy().prune_last && mixer_->takes_rows;
        Activation x = input(c, *stream);
        Tensor y;
        {
            Span span(mixer_->trace_name());
            y = mixer_->forward(c, x, entry, nullptr, rows_only);
        }
        if (rows_only) {
            // nothing but the head reads the stream after this block: go on with the rows it wants
            c.sub_stream.reset(new Stream());
            Stream* sub = c.sub_stream.get();
            sub->of_last_rows = true;
            sub->h = c.alloc(F32, {c.n_last, stream->h.shape[1]});
            if (c.n_last == 0) return sub;
            k_gather_rows(c, stream->h, c.dev.last_rows, c.n_last, sub->h);
            stream = sub;
        }
        add_normed(c, *stream, y, mixer_out_norm_.get(), feed_forward_ != nullptr);
        if (!feed_forward_) return stream;
        x = input(c, *stream);
        {
            Span span(feed_forward_->trace_name());
            y = feed_forward_->forward(c, x, nullptr);
        }
        add_normed(c, *stream, y, ff_out_norm_.get(), !last);
        return stream;
    }

private:
    struct Role { std::string role, prefix; std::shared_ptr<Part> part; };

    // what a part reads: the stream in the activation type (float32 runs read the stream itself)
    Activation input(StepContext& c, Stream& s) {
        Activation a;
        const bool pending = s.pending.kind != Pending::Nothing;
        if (s.pending.kind == Pending::Sums) raise(TQE_ERR_STATE, "output_norm block: the block before left an unfinished product on the stream");
        if (!pending && c.act_dtype == F32) { a.x = s.h; return a; }
        if (!pending && s.copy_valid) { a.x = s.copy; return a; }
        Tensor copy = c.act_dtype == F32 ? Tensor() : c.alloc(c.act_dtype, {s.h.shape[0], s.h.shape[1]});
        K::norm_add((float*)s.h.data, pending ? s.pending.t.data : nullptr, c.act_dtype, nullptr, 0, 0.f, copy.data, (int)s.h.shape[0], (int)s.h.shape[1], c.stream);
        s.pending = Pending();
        s.invalidate();
        if (c.act_dtype == F32) { a.x = s.h; return a; }
        s.copy = copy;
        s.copy_valid = true;
        a.x = copy;
        return a;
    }
    // h += norm(y) in float32; the stream's copy in the activation type comes out of the same kernel where a part will read it
    void add_normed(StepContext& c, Stream& s, const Tensor& y, const Norm* norm, bool copy_wanted) {
        Span span(norm ? norm->trace_name() : "add");
        const int64_t n = s.h.shape[0], hidden = s.h.shape[1];
        if (y.shape[0] != n || y.cols() != hidden) raise(TQE_ERR_STATE, "output_norm block: a part returned %s for a stream of [%lld, %lld]", y.describe().c_str(), (long long)n, (long long)hidden);
        s.invalidate();
        Tensor copy;
        if (copy_wanted && c.act_dtype != F32) copy = c.alloc(c.act_dtype, {n, hidden});
        const Tensor* w = norm ? norm->fold_weight() : nullptr;
        if (norm && !w) raise(TQE_ERR_ARGUMENT, "output_norm block: norm kind '%s' offers no weight to the kernel that adds a normed output", norm->kind.c_str());
        K::norm_add((float*)s.h.data, y.data, y.dtype, w ? w->data : nullptr, w ? w->dtype : 0, norm ? norm->fold_eps() : 0.f, copy.data, (int)n, (int)hidden, c.stream);
        if (copy.defined()) { s.copy = copy; s.copy_valid = true; }
    }

    std::vector<Role> roles_;
    std::shared_ptr<Mixer> mixer_;
    std::shared_ptr<FeedForward> feed_forward_;
    std::shared_ptr<Norm> mixer_out_norm_, ff_out_norm_;
};

}  // namespace

void register_stream_parts() {
    register_kind("position", "pair_hash", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<PairHash>(s, e); });
    register_kind("feed_forward", "activated", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<Activated>(s, e); });
    register_kind("block", "output_norm", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<OutputNormBlock>(s, e); });
}

}  // namespace tq
