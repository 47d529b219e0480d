// Sizudra: a decoder whose layers are listed one by one in its configuration.  The token embedding
// is joined by an embedding of the hashed pair (previous token, token).  A layer adds the normed
// output of its mixer and then of its feed-forward to the stream; nothing is normed in front of a
// part.  Two mixers, both grouped-query attention with values of their own size, a norm of every
// query and key head, rotation of a head's first elements, and values mixed with those of the first
// layer that mixes: "attention" sees every earlier position through an ordinary softmax;
// "attention_2" caps its scores, sees a window plus the sequence's first positions, and has a sink
// per head in the softmax's denominator.  The feed-forward is dense (gelu_tanh(gate) * up), or
// routed experts of the form down(relu(up)^2) whose weights are the softmax over the chosen logits,
// with a shared expert behind a sigmoid gate per token; or absent.
//
// This file holds what is particular to the architecture: which config.json keys it reads and how
// they become a ModelSpec with the checkpoint's tensor names.  Nothing here computes.
//
// config.json: architecture "Sizudra"; vocab, width; embedding.bigram {buckets, mul_prev, mul_cur};
// norm.eps; layers: a list of {type, mixer, mlp}.  mixer: {heads, kv_heads, dim, vdim, scale,
// rot {base, dims}, v_mix (optional)}, and for attention_2 also softcap and mask {size, keep_first}.
// mlp: null, {kind "dense", ff}, or {kind "moe", router {experts, top}, expert {ff}, shared {ff}
// (optional)}.  max_positions (optional): the longest sequence, 131072 unless given.
// Tensors: embed, bigram, head, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.{q, k, v, o, q.norm,
// k.norm, vmix, sink}, l<i>.mlp.{gate, up, down} or l<i>.mlp.{router, e<j>.up, e<j>.down,
// shared.up, shared.down, shared.sg}.
#include <algorithm>

#include "config.h"

namespace tq {
namespace {

const long long DEFAULT_MAX_POSITIONS = 131072;

const Json& object_at(const Json& parent, const char* key, const std::string& where) {
    const Json& j = parent[key];
    if (!j.is_object()) raise(TQE_ERR_CONFIG, "%s: '%s' must be an object", where.c_str(), key);
    return j;
}

Json mixer_typed(const Json& raw, const std::string& where, bool second) {
    KeyReader r(raw, where);
    Json m = Json::object();
    m.set("heads", r.integer("heads", 1));
    m.set("kv_heads", r.integer("kv_heads", 1));
    m.set("dim", r.integer("dim", 1));
    m.set("vdim", r.integer("vdim", 1));
    m.set("scale", r.number("scale", true));
    if (m["heads"].as_int() % m["kv_heads"].as_int())
        raise(TQE_ERR_CONFIG, "%s: %lld heads are not a multiple of %lld kv_heads", where.c_str(), (long long)m["heads"].as_int(), (long long)m["kv_heads"].as_int());
    KeyReader rot(object_at(raw, "rot", where), where + ".rot");
    const long long dims = rot.integer("dims", 0);
    if (dims % 2 || dims > m["dim"].as_int()) raise(TQE_ERR_CONFIG, "%s.rot: dims %lld must be even and at most dim %lld", where.c_str(), dims, (long long)m["dim"].as_int());
    m.set("rot_base", rot.number("base", true));
    m.set("rot_dims", dims);
    m.set("v_mix", r.boolean_or("v_mix", false));
    if (second) {
        m.set("softcap", r.number("softcap", true));
        KeyReader mask(object_at(raw, "mask", where), where + ".mask");
        m.set("window", mask.integer("size", 1));
        m.set("keep_first", mask.integer_or("keep_first", 0, 0));
        if (m["window"].as_int() > 0x3fffffff || m["keep_first"].as_int() > 0x3fffffff) raise(TQE_ERR_CONFIG, "%s.mask: size or keep_first is out of range", where.c_str());
    } else {
        m.set("softcap", Json());
        m.set("window", Json());
        m.set("keep_first", 0);
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
        KeyReader router(object_at(raw, "router", where), where + ".router");
        const long long experts = router.integer("experts", 1), top = router.integer("top", 1);
        if (top > experts) raise(TQE_ERR_CONFIG, "%s.router: top %lld of %lld experts", where.c_str(), top, experts);
        m.set("experts", experts);
        m.set("top", top);
        m.set("expert_ff", KeyReader(object_at(raw, "expert", where), where + ".expert").integer("ff", 1));
        m.set("shared_ff", raw["shared"].is_null() ? Json() : Json(KeyReader(object_at(raw, "shared", where), where + ".shared").integer("ff", 1)));
    } else {
        raise(TQE_ERR_CONFIG, "%s: unknown kind '%s' (known: dense, moe)", where.c_str(), kind.c_str());
    }
    return m;
}

Json sizudra_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    Json c = Json::object();
    c.set("vocab", r.integer("vocab", 1));
    c.set("width", r.integer("width", 1));
    KeyReader big(object_at(object_at(raw, "embedding", where), "bigram", where + ": embedding"), where + ": embedding.bigram");
    c.set("bigram_buckets", big.integer("buckets", 1));
    c.set("bigram_mul_prev", big.integer("mul_prev", 0));
    c.set("bigram_mul_cur", big.integer("mul_cur", 0));
    c.set("norm_eps", KeyReader(object_at(raw, "norm", where), where + ": norm").number("eps"));
    c.set("max_positions", r.integer_or("max_positions", DEFAULT_MAX_POSITIONS, 1));
    if (!raw["layers"].is_array() || raw["layers"].items().empty()) raise(TQE_ERR_CONFIG, "%s: 'layers' must be a list of at least one layer", where.c_str());
    Json list = Json::array();
    long long i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string at = format("%s: layers[%lld]", where.c_str(), i++);
        if (!l.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object", at.c_str());
        const std::string type = KeyReader(l, at).string("type");
        if (type != "attention" && type != "attention_2") raise(TQE_ERR_CONFIG, "%s: unknown type '%s' (known: attention, attention_2)", at.c_str(), type.c_str());
        Json t = Json::object();
        t.set("type", type);
        t.set("mixer", mixer_typed(object_at(l, "mixer", at), at + ".mixer", type == "attention_2"));
        t.set("mlp", mlp_typed(l["mlp"], at + ".mlp"));
        list.push(t);
    }
    c.set("layers", list);
    // the layers that mix values all mix with the first of them: their values must be of one size
    const Json* first = nullptr;
    for (const Json& l : list.items()) {
        const Json& m = l["mixer"];
        if (!m["v_mix"].as_bool()) continue;
        if (!first) { first = &m; continue; }
        if (m["kv_heads"].as_int() != (*first)["kv_heads"].as_int() || m["vdim"].as_int() != (*first)["vdim"].as_int())
            raise(TQE_ERR_CONFIG, "%s: layers that mix values (v_mix) differ in kv_heads or vdim", where.c_str());
    }
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

ModelSpec sizudra_spec(const Json& c) {
    const long long width = c["width"].as_int();
    const PartSpec norm = part("rms_norm", {{"size", width}, {"eps", c["norm_eps"]}, {"tensor", ""}});
    ModelSpec s;
    s.architecture = "Sizudra";
    s.vocab_size = c["vocab"].as_int();
    s.hidden_size = width;
    s.max_positions = c["max_positions"].as_int();
    s.embedding_name = "embed";
    s.head_name = "head";
    s.stream_position = part("pair_hash", {{"hidden", width}, {"vocab", c["vocab"]}, {"buckets", c["bigram_buckets"]}, {"mul_prev", c["bigram_mul_prev"]},
                                           {"mul_cur", c["bigram_mul_cur"]}, {"max_positions", c["max_positions"]}, {"tensor", ""}});
    s.stream_position_prefix = "bigram";
    // Layers of equal head sizes and equal windows share a group of the cache, and the cache's bookkeeping takes TQE_MAX_GROUPS of
    // them: a model with more different windows than that keeps every page (what a layer sees is its own window still).
    std::vector<std::vector<long long>> distinct;
    for (const Json& layer : c["layers"].items()) {
        const Json& m = layer["mixer"];
        const std::vector<long long> key = {m["kv_heads"].as_int(), m["dim"].as_int(), m["vdim"].as_int(), m["window"].is_null() ? 0 : m["window"].as_int(),
                                            m["keep_first"].as_int()};
        if (std::find(distinct.begin(), distinct.end(), key) == distinct.end()) distinct.push_back(key);
    }
    const bool keep_all = (int)distinct.size() > TQE_MAX_GROUPS;
    bool mixing_begun = false;
    size_t l = 0;
    for (const Json& layer : c["layers"].items()) {
        const Json& m = layer["mixer"];
        const Json& mlp = layer["mlp"];
        const bool second = layer["type"].as_string() == "attention_2";
        const PartSpec position = m["rot_dims"].as_int() > 0
            ? part("rotary", {{"theta", m["rot_base"]}, {"rot_dim", m["rot_dims"]}, {"max_positions", c["max_positions"]}, {"style", "halves"}})
            : part("none", {{"max_positions", c["max_positions"]}});
        const char* value_mix = !m["v_mix"].as_bool() ? "none" : mixing_begun ? "mixed" : "source";
        if (m["v_mix"].as_bool()) mixing_begun = true;
        const PartSpec mixer = part("attention", {{"hidden", width}, {"n_heads", m["heads"]}, {"n_kv_heads", m["kv_heads"]}, {"head_dim", m["dim"]},
                                                  {"value_dim", m["vdim"]}, {"scale", m["scale"]}, {"qk_norm", true}, {"eps", c["norm_eps"]},
                                                  {"window", m["window"]}, {"keep_first", m["keep_first"]}, {"cache_keeps_all", keep_all}, {"cap", m["softcap"]}, {"sink", second},
                                                  {"value_mix", value_mix}, {"position", position.to_json()},
                                                  {"names", names_of({{"q", "q"}, {"k", "k"}, {"v", "v"}, {"o", "o"}, {"q_norm", "q.norm"}, {"k_norm", "k.norm"},
                                                                      {"sink", "sink"}, {"mix", "vmix"}})}});
        Json ff;
        if (!mlp.is_null()) {
            if (mlp["kind"].as_string() == "dense") {
                ff = part("gated", {{"hidden", width}, {"inter", mlp["ff"]}, {"gate", "gelu_tanh"}, {"names", names_of({{"gate", "gate"}, {"up", "up"}, {"down", "down"}})}}).to_json();
            } else {
                const Json shared = mlp["shared_ff"].is_null()
                    ? Json()
                    : part("activated", {{"hidden", width}, {"inter", mlp["shared_ff"]}, {"gate", "relu2"}, {"names", names_of({{"up", "up"}, {"down", "down"}})}}).to_json();
                ff = part("routed_experts", {{"hidden", width}, {"inter", mlp["expert_ff"]}, {"n_experts", mlp["experts"]}, {"top", mlp["top"]},
                                             {"router_scale", 1.0}, {"gate", "relu2"}, {"gated", false}, {"normalize", "chosen"}, {"shared", shared},
                                             {"shared_gate", mlp["shared_ff"].is_null() ? Json() : Json("shared.sg")}}).to_json();
            }
        }
        LayerSpec spec;
        spec.prefix = format("l%zu.", l);
        spec.block = part("output_norm", {{"mixer", mixer.to_json()}, {"feed_forward", ff}, {"mixer_out_norm", norm.to_json()},
                                          {"ff_out_norm", mlp.is_null() ? Json() : norm.to_json()},
                                          {"names", names_of({{"mixer", "mix."}, {"feed_forward", "mlp."}, {"mixer_out_norm", "norm1"}, {"ff_out_norm", "norm2"}})}});
        s.layers.push_back(spec);
        Run run;
        run.layer = (int)l++;
        s.order.push_back(run);
    }
    s.final_norm = norm;
    s.final_norm_prefix = "final.norm";
    return s;
}

}  // namespace

void register_sizudra() {
    Architecture a;
    a.name = "Sizudra";
    a.model_types = {"sizudra"};
    a.typed_config = sizudra_typed;
    a.build_spec = sizudra_spec;
    register_architecture(a);
}

}  // namespace tq
