// gl3_modeldir.cpp — host-only loader of model folders: config.json picks the model class from the table of registered designs and
// gives every size; model.safetensors (8-byte little-endian header length, a JSON header name -> {dtype, shape, data_offsets}, then
// the data) is mmap'd and every tensor goes from the mapping to gl3_upload_tensor under the id its name maps to.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../include/gpullama3_hip.h"

void gl3_set_create_error(const char* msg);          // the message gl3_last_error(NULL) returns (gl3_api.hip)

namespace {

std::string g_dir_err;

// ---- a small JSON reader (objects keep their key order) ---------------------------------------------------------------------------
struct JVal {
    enum Kind { NUL, BOOL, NUM, STR, ARR, OBJ } kind = NUL;
    bool b = false;
    double num = 0;
    std::string str;
    std::vector<JVal> arr;
    std::vector<std::pair<std::string, JVal>> obj;
    const JVal* get(const char* key) const {
        if (kind != OBJ) return nullptr;
        for (auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool is_null() const { return kind == NUL; }
};

struct JParser {
    const char* p; const char* e; std::string err; int depth = 0;
    void ws() { while (p < e && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
    bool fail(const char* m) { if (err.empty()) err = m; return false; }
    bool parse_string(std::string& out) {
        if (p >= e || *p != '"') return fail("json: expected a string");
        ++p;
        while (p < e && *p != '"') {
            if (*p == '\\') {
                if (++p >= e) return fail("json: bad escape");
                switch (*p) {
                    case 'n': out += '\n'; break; case 't': out += '\t'; break; case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break; case 'f': out += '\f'; break;
                    case 'u': {
                        if (e - p < 5) return fail("json: bad \\u escape");
                        unsigned v = (unsigned)strtoul(std::string(p + 1, p + 5).c_str(), nullptr, 16);
                        if (v < 0x80) out += (char)v;
                        else if (v < 0x800) { out += (char)(0xC0 | (v >> 6)); out += (char)(0x80 | (v & 0x3F)); }
                        else { out += (char)(0xE0 | (v >> 12)); out += (char)(0x80 | ((v >> 6) & 0x3F)); out += (char)(0x80 | (v & 0x3F)); }
                        p += 4;
                        break;
                    }
                    default: out += *p;
                }
                ++p;
            } else
                out += *p++;
        }
        if (p >= e) return fail("json: unterminated string");
        ++p;
        return true;
    }
    bool parse(JVal& v) {
        if (++depth > 64) return fail("json: nested too deeply");
        ws();
        if (p >= e) return fail("json: unexpected end");
        bool ok = true;
        if (*p == '{') {
            v.kind = JVal::OBJ; ++p; ws();
            if (p < e && *p == '}') ++p;
            else
                for (;;) {
                    ws();
                    std::string k;
                    if (!parse_string(k)) { ok = false; break; }
                    ws();
                    if (p >= e || *p != ':') { ok = fail("json: expected ':'"); break; }
                    ++p;
                    v.obj.emplace_back(k, JVal());
                    if (!parse(v.obj.back().second)) { ok = false; break; }
                    ws();
                    if (p < e && *p == ',') { ++p; continue; }
                    if (p < e && *p == '}') { ++p; break; }
                    ok = fail("json: expected ',' or '}'"); break;
                }
        } else if (*p == '[') {
            v.kind = JVal::ARR; ++p; ws();
            if (p < e && *p == ']') ++p;
            else
                for (;;) {
                    v.arr.emplace_back();
                    if (!parse(v.arr.back())) { ok = false; break; }
                    ws();
                    if (p < e && *p == ',') { ++p; continue; }
                    if (p < e && *p == ']') { ++p; break; }
                    ok = fail("json: expected ',' or ']'"); break;
                }
        } else if (*p == '"') {
            v.kind = JVal::STR; ok = parse_string(v.str);
        } else if (e - p >= 4 && !strncmp(p, "true", 4)) { v.kind = JVal::BOOL; v.b = true; p += 4; }
        else if (e - p >= 5 && !strncmp(p, "false", 5)) { v.kind = JVal::BOOL; v.b = false; p += 5; }
        else if (e - p >= 4 && !strncmp(p, "null", 4)) { v.kind = JVal::NUL; p += 4; }
        else {
            const char* s = p;
            while (p < e && (strchr("+-.eE", *p) || (*p >= '0' && *p <= '9'))) ++p;
            if (p == s) ok = fail("json: unexpected character");
            else { v.kind = JVal::NUM; v.num = strtod(std::string(s, p).c_str(), nullptr); }
        }
        --depth;
        return ok;
    }
};

bool parse_json(const char* data, size_t n, JVal& out, std::string& err) {
    JParser ps{data, data + n, {}};
    if (!ps.parse(out)) { err = ps.err; return false; }
    return true;
}

bool read_file(const std::string& path, std::string& out) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return false;
    char buf[65536];
    size_t n;
    while ((n = fread(buf, 1, sizeof buf, f)) > 0) out.append(buf, n);
    fclose(f);
    return true;
}

bool get_int(const JVal& o, const char* key, int32_t& out, std::string& err, bool required = true) {
    const JVal* v = o.get(key);
    if (!v || v->kind != JVal::NUM) { if (required) err = std::string("config: missing number '") + key + "'"; return false; }
    if (v->num != std::floor(v->num) || std::fabs(v->num) > 2e9) { err = std::string("config: '") + key + "' is not a 32-bit integer"; return false; }
    out = (int32_t)v->num;
    return true;
}
bool get_float(const JVal& o, const char* key, float& out, std::string& err) {
    const JVal* v = o.get(key);
    if (!v || v->kind != JVal::NUM) { err = std::string("config: missing number '") + key + "'"; return false; }
    out = (float)v->num;
    return true;
}

// ---- registered designs -----------------------------------------------------------------------------------------------------------
// what a description points to besides the layer list (second mixers, decay lists): lives until gl3_create has copied it
struct DescStore { std::deque<gl3_layer_desc> descs; std::deque<std::vector<float>> floats; };
struct Design {
    const char* architecture;                                  // config.json "architecture"
    bool (*describe)(const JVal& cfg, gl3_model_desc& d, std::vector<gl3_layer_desc>& layers, DescStore& store, std::string& err);
    // false: not a tensor of this design.  expert >= 0: the tensor is one expert's part of the stacked tensor `id` ([experts][..]); the
    // loader puts the parts together and uploads the whole once all of them are there
    bool (*tensor)(const std::string& name, int32_t& id, int32_t& layer, int32_t& expert);
};

// Noditar: a list of layers of three mixer types behind hyper-connected residual streams.  The design fixes: unit-RMS q and k, distance
// slopes 2^(-8 (h + 1) / H), one extra unit in the attention softmax's denominator (not in the latent attention's), sigmoid output
// gates, and the feed-forward activation g sigmoid(1.702 g) (u + 1).
bool noditar_describe(const JVal& cfg, gl3_model_desc& d, std::vector<gl3_layer_desc>& layers, DescStore&, std::string& err) {
    d.arch = GL3_ARCH_NODITAR;
    d.weight_type = GL3_TYPE_BF16;
    if (!get_int(cfg, "vocab", d.vocab, err) || !get_int(cfg, "width", d.dim, err)) return false;
    d.streams = 1;
    if (cfg.get("streams") && !get_int(cfg, "streams", d.streams, err)) return false;
    const JVal* norm = cfg.get("norm");
    if (!norm || !get_float(*norm, "eps", d.rms_eps, err)) { if (err.empty()) err = "config: missing norm.eps"; return false; }
    const JVal* ls = cfg.get("layers");
    if (!ls || ls->kind != JVal::ARR || ls->arr.empty()) { err = "config: 'layers' must be a non-empty list"; return false; }
    for (const JVal& l : ls->arr) {
        gl3_layer_desc ld{};
        const JVal *ty = l.get("type"), *mx = l.get("mixer"), *mlp = l.get("mlp");
        if (!ty || ty->kind != JVal::STR || !mx || mx->kind != JVal::OBJ) { err = "config: a layer needs 'type' and 'mixer'"; return false; }
        if (!get_int(*mx, "heads", ld.heads, err) || !get_int(*mx, "vdim", ld.vdim, err)) return false;
        ld.kv_heads = ld.heads;
        ld.out_gate = 1;
        if (ty->str == "attention") {
            ld.mixer = GL3_MIX_ATTENTION;
            if (!get_int(*mx, "kv_heads", ld.kv_heads, err) || !get_int(*mx, "dim", ld.dim, err) || !get_float(*mx, "scale", ld.scale, err)) return false;
            ld.qk_unit_norm = 1; ld.slope_log2 = 8.f; ld.softmax_sink = 1;
        } else if (ty->str == "latent_attention") {
            ld.mixer = GL3_MIX_LATENT;
            if (!get_int(*mx, "dim", ld.dim, err) || !get_int(*mx, "kv_rank", ld.kv_rank, err) || !get_float(*mx, "scale", ld.scale, err)) return false;
        } else if (ty->str == "mamba2") {
            ld.mixer = GL3_MIX_SSM;
            ld.out_gate = 0;
            if (!get_int(*mx, "conv", ld.conv, err) || !get_int(*mx, "groups", ld.groups, err) || !get_int(*mx, "norm_groups", ld.norm_groups, err) ||
                !get_int(*mx, "state", ld.state, err))
                return false;
        } else { err = "config: unknown layer type '" + ty->str + "'"; return false; }
        if (mlp && !mlp->is_null()) {
            const JVal* kind = mlp->get("kind");
            if (!kind || kind->kind != JVal::STR || kind->str != "dense") { err = "config: mlp.kind must be 'dense'"; return false; }
            if (!get_int(*mlp, "ff", ld.ff, err) || !get_float(*mlp, "limit", ld.ff_limit, err)) return false;
            ld.ff_alpha = 1.702f; ld.ff_shift = 1.f;
        }
        layers.push_back(ld);
    }
    d.n_layers = (int32_t)layers.size();
    return true;
}

// "l<digits>.<leaf>" -> layer and leaf; false for any other name
bool split_layer_name(const std::string& name, int32_t& layer, std::string& leaf) {
    if (name.size() < 4 || name[0] != 'l') return false;
    size_t i = 1;
    while (i < name.size() && name[i] >= '0' && name[i] <= '9') ++i;
    if (i == 1 || i > 8 || i >= name.size() || name[i] != '.') return false;
    layer = atoi(name.substr(1, i - 1).c_str());
    leaf = name.substr(i + 1);
    return true;
}

bool noditar_tensor(const std::string& name, int32_t& id, int32_t& layer, int32_t& expert) {
    expert = -1;
    static const std::map<std::string, int> global = {{"embed", GL3_T_TOKEN_EMBD}, {"head", GL3_T_OUTPUT}, {"final.norm", GL3_T_OUTPUT_NORM}};
    static const std::map<std::string, int> leaf = {
        {"norm1", GL3_T_ATTN_NORM}, {"norm2", GL3_T_FFN_NORM}, {"mix.q", GL3_T_WQ}, {"mix.k", GL3_T_WK}, {"mix.v", GL3_T_WV}, {"mix.g", GL3_T_ATTN_GATE},
        {"mix.o", GL3_T_WO}, {"mix.dkv", GL3_T_KV_DOWN}, {"mix.dkv.norm", GL3_T_KV_DOWN_NORM}, {"mix.uk", GL3_T_K_UP}, {"mix.uv", GL3_T_V_UP},
        {"mix.in", GL3_T_SSM_IN}, {"mix.conv", GL3_T_SSM_CONV}, {"mix.conv.b", GL3_T_SSM_CONV_BIAS}, {"mix.dt_bias", GL3_T_SSM_DT_BIAS},
        {"mix.A_log", GL3_T_SSM_A_LOG}, {"mix.D", GL3_T_SSM_D}, {"mix.norm", GL3_T_SSM_NORM}, {"mlp.gate", GL3_T_W1}, {"mlp.up", GL3_T_W3},
        {"mlp.down", GL3_T_W2}, {"hc1.in", GL3_T_HC1_IN}, {"hc1.out", GL3_T_HC1_OUT}, {"hc1.mix", GL3_T_HC1_MIX}, {"hc2.in", GL3_T_HC2_IN},
        {"hc2.out", GL3_T_HC2_OUT}, {"hc2.mix", GL3_T_HC2_MIX}};
    auto g = global.find(name);
    if (g != global.end()) { id = g->second; layer = 0; return true; }
    std::string lf;
    if (!split_layer_name(name, layer, lf)) return false;
    auto f = leaf.find(lf);
    if (f == leaf.end()) return false;
    id = f->second;
    return true;
}

// Vonulix: attention layers on one plain residual stream.  config.json gives every size and the constants that differ between models
// (embedding scale, rotary base / dims / position scaling, score scale, window and kept first keys, clip limits, expert counts); the
// design fixes: norm weights kept as their deviation from one (weight = 1 + stored value), unit-RMS values, values rotated by their position and outputs
// turned back, one sigmoid output gate per head, sigmoid router scores that scale the chosen experts' inputs, the expert activation
// g sigmoid(1.702 g) (u + 1), a gated shared expert, a per-layer token input and the weighted average over all earlier layers' results.
bool vonulix_describe(const JVal& cfg, gl3_model_desc& d, std::vector<gl3_layer_desc>& layers, DescStore&, std::string& err) {
    d.arch = GL3_ARCH_LAYERLIST;
    d.weight_type = GL3_TYPE_BF16;
    if (!get_int(cfg, "vocab", d.vocab, err) || !get_int(cfg, "width", d.dim, err)) return false;
    d.streams = 0;
    d.norm_offset = 1.f;
    d.depth_mix = 1;
    d.embedding_scale = 1.f;
    if (const JVal* e = cfg.get("embedding"))
        if (e->kind == JVal::OBJ && e->get("scale") && !get_float(*e, "scale", d.embedding_scale, err)) return false;
    if (const JVal* ts = cfg.get("token_side"))
        if (ts->kind == JVal::OBJ && !get_int(*ts, "dim", d.side_dim, err)) return false;
    const JVal* norm = cfg.get("norm");
    if (!norm || !get_float(*norm, "eps", d.rms_eps, err)) { if (err.empty()) err = "config: missing norm.eps"; return false; }
    const JVal* ls = cfg.get("layers");
    if (!ls || ls->kind != JVal::ARR || ls->arr.empty()) { err = "config: 'layers' must be a non-empty list"; return false; }
    for (const JVal& l : ls->arr) {
        gl3_layer_desc ld{};
        const JVal *ty = l.get("type"), *mx = l.get("mixer"), *mlp = l.get("mlp");
        if (!ty || ty->kind != JVal::STR || !mx || mx->kind != JVal::OBJ) { err = "config: a layer needs 'type' and 'mixer'"; return false; }
        if (ty->str != "attention") { err = "config: unknown layer type '" + ty->str + "'"; return false; }
        ld.mixer = GL3_MIX_ATTENTION;
        if (!get_int(*mx, "heads", ld.heads, err) || !get_int(*mx, "kv_heads", ld.kv_heads, err) || !get_int(*mx, "dim", ld.dim, err) ||
            !get_int(*mx, "vdim", ld.vdim, err) || !get_float(*mx, "scale", ld.scale, err))
            return false;
        ld.out_gate = 2; ld.v_unit_norm = 1; ld.v_rot = 1;
        const JVal* rot = mx->get("rot");
        if (!rot || rot->kind != JVal::OBJ || !get_int(*rot, "dims", ld.rot_dims, err) || !get_float(*rot, "base", ld.rot_base, err)) {
            if (err.empty()) err = "config: an attention mixer needs rot.dims and rot.base";
            return false;
        }
        ld.rot_divide = 1.f;
        if (const JVal* sc = rot->get("scaling"))
            if (sc->kind == JVal::OBJ && !get_float(*sc, "factor", ld.rot_divide, err)) return false;
        if (const JVal* mask = mx->get("mask"))
            if (mask->kind == JVal::OBJ) {
                if (!get_int(*mask, "size", ld.window, err)) return false;
                if (mask->get("keep_first") && !get_int(*mask, "keep_first", ld.keep_first, err)) return false;
            }
        if (mlp && !mlp->is_null()) {
            const JVal *kind = mlp->get("kind"), *ex = mlp->get("expert"), *ro = mlp->get("router"), *sh = mlp->get("shared");
            if (!kind || kind->kind != JVal::STR || kind->str != "moe") { err = "config: mlp.kind must be 'moe'"; return false; }
            if (!ex || !ro || !get_int(*ex, "ff", ld.ff, err) || !get_float(*ex, "limit", ld.ff_limit, err) || !get_int(*ro, "experts", ld.experts, err) ||
                !get_int(*ro, "top", ld.top, err)) {
                if (err.empty()) err = "config: a mixture of experts needs 'expert' and 'router'";
                return false;
            }
            if (sh && !sh->is_null() && (!get_int(*sh, "ff", ld.shared_ff, err) || !get_float(*sh, "limit", ld.shared_limit, err))) return false;
            ld.ff_alpha = 1.702f; ld.ff_shift = 1.f;
        }
        layers.push_back(ld);
    }
    d.n_layers = (int32_t)layers.size();
    return true;
}

bool vonulix_tensor(const std::string& name, int32_t& id, int32_t& layer, int32_t& expert) {
    static const std::map<std::string, int> global = {{"embed", GL3_T_TOKEN_EMBD}, {"head", GL3_T_OUTPUT}, {"final.norm", GL3_T_OUTPUT_NORM},
                                                      {"side.embed", GL3_T_SIDE_EMBD}};
    static const std::map<std::string, int> leaf = {
        {"norm1", GL3_T_ATTN_NORM}, {"norm2", GL3_T_FFN_NORM}, {"mix.q", GL3_T_WQ}, {"mix.k", GL3_T_WK}, {"mix.v", GL3_T_WV}, {"mix.g", GL3_T_ATTN_GATE},
        {"mix.o", GL3_T_WO}, {"mlp.router", GL3_T_FFN_GATE_INP}, {"mlp.shared.gate", GL3_T_W1}, {"mlp.shared.up", GL3_T_W3}, {"mlp.shared.down", GL3_T_W2},
        {"mlp.shared.sg", GL3_T_FFN_GATE_INP_SHEXP}, {"dwa", GL3_T_DEPTH_MIX}, {"side.gate", GL3_T_SIDE_GATE}, {"side.proj", GL3_T_SIDE_PROJ},
        {"side.norm", GL3_T_SIDE_NORM}};
    static const std::map<std::string, int> part = {{"gate", GL3_T_FFN_GATE_EXPS}, {"up", GL3_T_FFN_UP_EXPS}, {"down", GL3_T_FFN_DOWN_EXPS}};
    expert = -1;
    auto g = global.find(name);
    if (g != global.end()) { id = g->second; layer = 0; return true; }
    std::string lf;
    if (!split_layer_name(name, layer, lf)) return false;
    auto f = leaf.find(lf);
    if (f != leaf.end()) { id = f->second; return true; }
    if (lf.compare(0, 5, "mlp.e") == 0) {          // mlp.e<k>.gate | up | down
        size_t i = 5;
        while (i < lf.size() && lf[i] >= '0' && lf[i] <= '9') ++i;
        if (i == 5 || i > 12 || i >= lf.size() || lf[i] != '.') return false;
        auto pf = part.find(lf.substr(i + 1));
        if (pf == part.end()) return false;
        id = pf->second; expert = atoi(lf.substr(5, i - 5).c_str());
        return true;
    }
    return false;
}

// Kosusun: every layer is a parallel block — one RMS norm, whose output feeds the mixer and the feed-forward alike, and
// x <- x + residual_mult (mixer + feed-forward).  Two layer types.  "parallel": two mixers side by side, `left` = grouped-query attention
// (biased q / k / v, RMS norm with weights over the whole q and the whole k projection, interleaved rotary pairs with linear position
// scaling, a sliding window plus one averaged key / value per finished run of `mask.pool` positions behind it, a learned sink logit per
// head) and `right` = retention (a matrix memory with a fixed decay per head, half-split rotary pairs, keys times dim^(-1/2), unit-RMS
// heads times silu(W_g h)), added as left_scale * left + right_scale * right.  "mlstm": a matrix memory with exponential gates
// (capped log gates, running maximum, normaliser; queries times dim^(-1/2); unit-RMS heads with a weight, times sigmoid(W_g h)).  The
// feed-forward is gelu_tanh(W_gate h) * (W_up h) through W_down.  config.json gives every size and the constants named above; the
// rest (the forms of the norms, gates and activations) is the design's and is fixed here.
bool get_rot(const JVal& mx, gl3_layer_desc& ld, std::string& err) {
    const JVal* rot = mx.get("rot");
    if (!rot || rot->is_null()) return true;                 // no rotary positions
    if (rot->kind != JVal::OBJ || !get_int(*rot, "dims", ld.rot_dims, err) || !get_float(*rot, "base", ld.rot_base, err)) {
        if (err.empty()) err = "config: rot needs dims and base";
        return false;
    }
    ld.rot_divide = 1.f;
    if (const JVal* sc = rot->get("scaling"))
        if (sc->kind == JVal::OBJ && !get_float(*sc, "factor", ld.rot_divide, err)) return false;
    return true;
}
bool kosusun_attention(const JVal& mx, gl3_layer_desc& ld, std::string& err) {
    ld.mixer = GL3_MIX_ATTENTION;
    if (!get_int(mx, "heads", ld.heads, err) || !get_int(mx, "kv_heads", ld.kv_heads, err) || !get_int(mx, "dim", ld.dim, err) || !get_int(mx, "vdim", ld.vdim, err) ||
        !get_float(mx, "scale", ld.scale, err) || !get_rot(mx, ld, err))
        return false;
    ld.qk_bias = 1; ld.qk_unit_norm = 2; ld.rot_interleaved = 1; ld.softmax_sink = 2;
    if (const JVal* mask = mx.get("mask"))
        if (mask->kind == JVal::OBJ) {
            if (!get_int(*mask, "size", ld.window, err)) return false;
            if (mask->get("pool") && !get_int(*mask, "pool", ld.pool, err)) return false;
        }
    return true;
}
bool kosusun_retention(const JVal& mx, gl3_layer_desc& ld, DescStore& store, std::string& err) {
    ld.mixer = GL3_MIX_MEMORY;
    ld.mem_gates = GL3_MEM_DECAY;
    if (!get_int(mx, "heads", ld.heads, err) || !get_int(mx, "dim", ld.dim, err) || !get_int(mx, "vdim", ld.vdim, err) || !get_rot(mx, ld, err)) return false;
    ld.kv_heads = ld.heads;
    const JVal* dec = mx.get("decay");
    if (!dec || dec->kind != JVal::ARR || (int)dec->arr.size() != ld.heads) { err = "config: retention needs a decay per head"; return false; }
    store.floats.emplace_back();
    for (const JVal& v : dec->arr) {
        if (v.kind != JVal::NUM) { err = "config: decay must be numbers"; return false; }
        store.floats.back().push_back((float)v.num);
    }
    ld.mem_decay = store.floats.back().data();
    ld.mem_k_mul = (float)(1.0 / std::sqrt((double)std::max(1, ld.dim)));
    ld.mem_gate_act = 0; ld.mem_norm_weight = 0;
    return true;
}
bool kosusun_describe(const JVal& cfg, gl3_model_desc& d, std::vector<gl3_layer_desc>& layers, DescStore& store, std::string& err) {
    d.arch = GL3_ARCH_LAYERLIST;
    d.weight_type = GL3_TYPE_BF16;
    if (!get_int(cfg, "vocab", d.vocab, err) || !get_int(cfg, "width", d.dim, err)) return false;
    d.streams = 0;
    d.parallel_block = 1;
    d.embedding_scale = d.residual_scale = d.logit_scale = 1.f;
    if (const JVal* e = cfg.get("embedding"))
        if (e->kind == JVal::OBJ && e->get("scale") && !get_float(*e, "scale", d.embedding_scale, err)) return false;
    if (cfg.get("residual_mult") && !get_float(cfg, "residual_mult", d.residual_scale, err)) return false;
    if (cfg.get("logit_scale") && !get_float(cfg, "logit_scale", d.logit_scale, err)) return false;
    const JVal* norm = cfg.get("norm");
    if (!norm || !get_float(*norm, "eps", d.rms_eps, err)) { if (err.empty()) err = "config: missing norm.eps"; return false; }
    const JVal* ls = cfg.get("layers");
    if (!ls || ls->kind != JVal::ARR || ls->arr.empty()) { err = "config: 'layers' must be a non-empty list"; return false; }
    for (const JVal& l : ls->arr) {
        gl3_layer_desc ld{};
        const JVal *ty = l.get("type"), *mx = l.get("mixer"), *mlp = l.get("mlp");
        if (!ty || ty->kind != JVal::STR || !mx || mx->kind != JVal::OBJ) { err = "config: a layer needs 'type' and 'mixer'"; return false; }
        if (ty->str == "parallel") {
            const JVal *left = mx->get("left"), *right = mx->get("right");
            if (!left || left->kind != JVal::OBJ || !right || right->kind != JVal::OBJ) { err = "config: a parallel mixer needs 'left' and 'right'"; return false; }
            gl3_layer_desc rd{};
            if (!kosusun_attention(*left, ld, err) || !kosusun_retention(*right, rd, store, err)) return false;
            ld.out_scale = rd.out_scale = 1.f;
            if (mx->get("left_scale") && !get_float(*mx, "left_scale", ld.out_scale, err)) return false;
            if (mx->get("right_scale") && !get_float(*mx, "right_scale", rd.out_scale, err)) return false;
            if (ld.out_scale == 0.f || rd.out_scale == 0.f) { err = "config: left_scale and right_scale must not be zero"; return false; }
            store.descs.push_back(rd);
            ld.beside = &store.descs.back();
        } else if (ty->str == "mlstm") {
            ld.mixer = GL3_MIX_MEMORY;
            ld.mem_gates = GL3_MEM_EXP_GATES;
            if (!get_int(*mx, "heads", ld.heads, err) || !get_int(*mx, "dim", ld.dim, err) || !get_int(*mx, "vdim", ld.vdim, err) ||
                !get_float(*mx, "gate_cap", ld.mem_gate_cap, err))
                return false;
            ld.kv_heads = ld.heads;
            ld.mem_q_mul = (float)(1.0 / std::sqrt((double)std::max(1, ld.dim)));
            ld.mem_gate_act = 1; ld.mem_norm_weight = 1;
        } else { err = "config: unknown layer type '" + ty->str + "'"; return false; }
        if (mlp && !mlp->is_null()) {
            const JVal* kind = mlp->get("kind");
            if (!kind || kind->kind != JVal::STR || kind->str != "dense") { err = "config: mlp.kind must be 'dense'"; return false; }
            if (!get_int(*mlp, "ff", ld.ff, err)) return false;
            ld.ff_act = 1;
        }
        layers.push_back(ld);
    }
    d.n_layers = (int32_t)layers.size();
    return true;
}

bool kosusun_tensor(const std::string& name, int32_t& id, int32_t& layer, int32_t& expert) {
    static const std::map<std::string, int> global = {{"embed", GL3_T_TOKEN_EMBD}, {"head", GL3_T_OUTPUT}, {"final.norm", GL3_T_OUTPUT_NORM}};
    static const std::map<std::string, int> leaf = {{"norm1", GL3_T_ATTN_NORM}, {"mlp.gate", GL3_T_W1}, {"mlp.up", GL3_T_W3}, {"mlp.down", GL3_T_W2}};
    // tensors of one mixer, after "mix." (mlstm), "mix.left." (attention) or "mix.right." (retention)
    static const std::map<std::string, int> mix = {
        {"q", GL3_T_WQ}, {"k", GL3_T_WK}, {"v", GL3_T_WV}, {"o", GL3_T_WO}, {"g", GL3_T_ATTN_GATE}, {"q.b", GL3_T_BQ}, {"k.b", GL3_T_BK}, {"v.b", GL3_T_BV},
        {"q.norm", GL3_T_ATTN_Q_NORM}, {"k.norm", GL3_T_ATTN_K_NORM}, {"sink", GL3_T_ATTN_SINK}, {"norm", GL3_T_SSM_NORM}, {"i", GL3_T_MEM_IGATE},
        {"f", GL3_T_MEM_FGATE}, {"i.b", GL3_T_MEM_IGATE_BIAS}, {"f.b", GL3_T_MEM_FGATE_BIAS}};
    expert = -1;
    auto g = global.find(name);
    if (g != global.end()) { id = g->second; layer = 0; return true; }
    std::string lf;
    if (!split_layer_name(name, layer, lf)) return false;
    auto f = leaf.find(lf);
    if (f != leaf.end()) { id = f->second; return true; }
    if (lf.compare(0, 4, "mix.") != 0) return false;
    std::string rest = lf.substr(4);
    if (rest.compare(0, 5, "left.") == 0) rest = rest.substr(5);
    else if (rest.compare(0, 6, "right.") == 0) { rest = rest.substr(6); layer |= GL3_LAYER_BESIDE; }
    auto m = mix.find(rest);
    if (m == mix.end()) return false;
    id = m->second;
    return true;
}

// Kugadra: one plain residual stream with a norm in front of AND behind every sublayer, x <- x + rms_norm(sublayer(rms_norm(x, w)), w_post).
// Two layer types.  "lightning": a matrix memory with a fixed decay per head behind silu-activated q / k / v (no rotation, no other
// scale), the heads side by side through ONE RMS norm with a weight, times sigmoid(W_g h).  "latent_attention": queries through a normed
// latent of their own, keys and values expanded from a cached normed latent, a rotated part of rot_dim entries per query head and one
// rotated key part for all heads (half-split pairs, frequencies blended towards / factor along a ramp over the pair index, cos and sin
// times 0.1 ln(factor) + 1), causal softmax, one sigmoid gate per head; a layer with "kv_from" reads that layer's cache.  Feed-forward:
// dense = W_down relu(W_up h)^2, or a mixture of silu-gated experts (softmax scores over all experts, chosen by score + a correction,
// weights = the chosen scores renormalised (+ 1e-20) times router.scale, applied to the experts' outputs) plus an ungated shared
// expert.  The head is the embedding table; logits pass cap * tanh(. / cap).  config.json gives every size and the constants named
// here; the forms are the design's and are fixed here.
bool kugadra_describe(const JVal& cfg, gl3_model_desc& d, std::vector<gl3_layer_desc>& layers, DescStore& store, std::string& err) {
    d.arch = GL3_ARCH_LAYERLIST;
    d.weight_type = GL3_TYPE_BF16;
    if (!get_int(cfg, "vocab", d.vocab, err) || !get_int(cfg, "width", d.dim, err)) return false;
    d.streams = 0;
    d.post_norms = 1;
    d.embedding_scale = 1.f;
    if (const JVal* e = cfg.get("embedding"))
        if (e->kind == JVal::OBJ && e->get("scale") && !get_float(*e, "scale", d.embedding_scale, err)) return false;
    if (const JVal* cap = cfg.get("logit_softcap"))
        if (!cap->is_null() && !get_float(cfg, "logit_softcap", d.logit_softcap, err)) return false;
    const JVal* norm = cfg.get("norm");
    if (!norm || !get_float(*norm, "eps", d.rms_eps, err)) { if (err.empty()) err = "config: missing norm.eps"; return false; }
    const JVal* ls = cfg.get("layers");
    if (!ls || ls->kind != JVal::ARR || ls->arr.empty()) { err = "config: 'layers' must be a non-empty list"; return false; }
    for (const JVal& l : ls->arr) {
        gl3_layer_desc ld{};
        const JVal *ty = l.get("type"), *mx = l.get("mixer"), *mlp = l.get("mlp");
        if (!ty || ty->kind != JVal::STR || !mx || mx->kind != JVal::OBJ) { err = "config: a layer needs 'type' and 'mixer'"; return false; }
        if (!get_int(*mx, "heads", ld.heads, err) || !get_int(*mx, "dim", ld.dim, err) || !get_int(*mx, "vdim", ld.vdim, err)) return false;
        ld.kv_heads = ld.heads;
        if (ty->str == "lightning") {
            ld.mixer = GL3_MIX_MEMORY;
            ld.mem_gates = GL3_MEM_DECAY;
            const JVal* dec = mx->get("decay");
            if (!dec || dec->kind != JVal::ARR || (int)dec->arr.size() != ld.heads) { err = "config: lightning needs a decay per head"; return false; }
            store.floats.emplace_back();
            for (const JVal& v : dec->arr) {
                if (v.kind != JVal::NUM) { err = "config: decay must be numbers"; return false; }
                store.floats.back().push_back((float)v.num);
            }
            ld.mem_decay = store.floats.back().data();
            ld.mem_qkv_act = 1; ld.mem_norm_whole = 1; ld.mem_norm_weight = 1; ld.mem_gate_act = 1;
        } else if (ty->str == "latent_attention") {
            ld.mixer = GL3_MIX_LATENT;
            ld.out_gate = 2;
            if (!get_int(*mx, "kv_rank", ld.kv_rank, err) || !get_int(*mx, "q_rank", ld.q_rank, err) || !get_float(*mx, "scale", ld.scale, err)) return false;
            if (mx->get("rot_dim") && !mx->get("rot_dim")->is_null() && !get_int(*mx, "rot_dim", ld.rot_dim, err)) return false;
            if (ld.q_rank < 1) { err = "config: q_rank must be positive"; return false; }
            if (const JVal* kf = mx->get("kv_from"))
                if (!kf->is_null()) {
                    int32_t j = -1;
                    if (!get_int(*mx, "kv_from", j, err)) return false;
                    if (j < 0 || j >= (int32_t)layers.size()) { err = "config: kv_from must name an earlier layer"; return false; }
                    ld.kv_share = j + 1;
                }
            if (ld.rot_dim > 0) {
                const JVal* rot = mx->get("rot");
                int32_t dims = 0;
                if (!rot || rot->kind != JVal::OBJ || !get_int(*rot, "dims", dims, err) || !get_float(*rot, "base", ld.rot_base, err)) {
                    if (err.empty()) err = "config: a latent attention with rot_dim needs rot.dims and rot.base";
                    return false;
                }
                if (dims != ld.rot_dim) { err = "config: rot.dims must equal rot_dim"; return false; }
                if (const JVal* sc = rot->get("scaling"))
                    if (sc->kind == JVal::OBJ &&
                        (!get_float(*sc, "factor", ld.rot_yarn_factor, err) || !get_float(*sc, "original", ld.rot_yarn_original, err) ||
                         !get_float(*sc, "fast", ld.rot_yarn_fast, err) || !get_float(*sc, "slow", ld.rot_yarn_slow, err)))
                        return false;
            }
        } else { err = "config: unknown layer type '" + ty->str + "'"; return false; }
        if (mlp && !mlp->is_null()) {
            const JVal* kind = mlp->get("kind");
            if (!kind || kind->kind != JVal::STR) { err = "config: mlp needs 'kind'"; return false; }
            if (kind->str == "dense") {
                if (!get_int(*mlp, "ff", ld.ff, err)) return false;
                ld.ff_act = 2;
            } else if (kind->str == "moe") {
                const JVal *ex = mlp->get("expert"), *ro = mlp->get("router"), *sh = mlp->get("shared");
                if (!ex || !ro || !get_int(*ex, "ff", ld.ff, err) || !get_int(*ro, "experts", ld.experts, err) || !get_int(*ro, "top", ld.top, err)) {
                    if (err.empty()) err = "config: a mixture of experts needs 'expert' and 'router'";
                    return false;
                }
                ld.route_scale = 1.f;
                if (ro->get("scale") && !get_float(*ro, "scale", ld.route_scale, err)) return false;
                if (sh && !sh->is_null() && !get_int(*sh, "ff", ld.shared_ff, err)) return false;
                ld.ff_alpha = 1.f; ld.ff_shift = 0.f;          // silu(g) u
                ld.route_softmax = 1; ld.route_bias = 1; ld.route_renorm = 1; ld.route_on_output = 1; ld.shared_ungated = 1;
            } else { err = "config: mlp.kind must be 'dense' or 'moe'"; return false; }
        }
        layers.push_back(ld);
    }
    d.n_layers = (int32_t)layers.size();
    return true;
}

bool kugadra_tensor(const std::string& name, int32_t& id, int32_t& layer, int32_t& expert) {
    static const std::map<std::string, int> global = {{"embed", GL3_T_TOKEN_EMBD}, {"final.norm", GL3_T_OUTPUT_NORM}};
    static const std::map<std::string, int> leaf = {
        {"norm1", GL3_T_ATTN_NORM}, {"norm2", GL3_T_FFN_NORM}, {"norm1b", GL3_T_ATTN_POST_NORM}, {"norm2b", GL3_T_FFN_POST_NORM},
        {"mix.q", GL3_T_WQ}, {"mix.k", GL3_T_WK}, {"mix.v", GL3_T_WV}, {"mix.g", GL3_T_ATTN_GATE}, {"mix.o", GL3_T_WO}, {"mix.norm", GL3_T_SSM_NORM},
        {"mix.dq", GL3_T_Q_DOWN}, {"mix.dq.norm", GL3_T_Q_DOWN_NORM}, {"mix.uq", GL3_T_WQ}, {"mix.dkv", GL3_T_KV_DOWN}, {"mix.dkv.norm", GL3_T_KV_DOWN_NORM},
        {"mix.uk", GL3_T_K_UP}, {"mix.uv", GL3_T_V_UP}, {"mlp.up", GL3_T_W3}, {"mlp.down", GL3_T_W2}, {"mlp.router", GL3_T_FFN_GATE_INP},
        {"mlp.correction", GL3_T_FFN_ROUTE_BIAS}, {"mlp.shared.gate", GL3_T_W1}, {"mlp.shared.up", GL3_T_W3}, {"mlp.shared.down", GL3_T_W2}};
    static const std::map<std::string, int> part = {{"gate", GL3_T_FFN_GATE_EXPS}, {"up", GL3_T_FFN_UP_EXPS}, {"down", GL3_T_FFN_DOWN_EXPS}};
    expert = -1;
    auto g = global.find(name);
    if (g != global.end()) { id = g->second; layer = 0; return true; }
    std::string lf;
    if (!split_layer_name(name, layer, lf)) return false;
    auto f = leaf.find(lf);
    if (f != leaf.end()) { id = f->second; return true; }
    if (lf.compare(0, 5, "mlp.e") == 0) {          // mlp.e<k>.gate | up | down
        size_t i = 5;
        while (i < lf.size() && lf[i] >= '0' && lf[i] <= '9') ++i;
        if (i == 5 || i > 12 || i >= lf.size() || lf[i] != '.') return false;
        auto pf = part.find(lf.substr(i + 1));
        if (pf == part.end()) return false;
        id = pf->second; expert = atoi(lf.substr(5, i - 5).c_str());
        return true;
    }
    return false;
}

const Design DESIGNS[] = {{"Noditar", noditar_describe, noditar_tensor}, {"Vonulix", vonulix_describe, vonulix_tensor}, {"Kosusun", kosusun_describe, kosusun_tensor},
                          {"Kugadra", kugadra_describe, kugadra_tensor}};

struct Mapping {
    void* p = MAP_FAILED; size_t n = 0;
    ~Mapping() { if (p != MAP_FAILED) munmap(p, n); }
};

}  // namespace

extern "C" {

int32_t gl3_is_model_dir(const char* path) {
    if (!path) return 0;
    struct stat st;
    if (stat(path, &st) != 0 || !S_ISDIR(st.st_mode)) return 0;
    return stat((std::string(path) + "/config.json").c_str(), &st) == 0 ? 1 : 0;
}

static int32_t load_model_dir(const char* dir, const gl3_model_desc* opts, gl3_ctx** out);
int32_t gl3_load_model_dir(const char* dir, const gl3_model_desc* opts, gl3_ctx** out) {
    const int32_t r = load_model_dir(dir, opts, out);
    if (r != GL3_OK) gl3_set_create_error(g_dir_err.c_str());
    return r;
}

static int32_t load_model_dir(const char* dir, const gl3_model_desc* opts, gl3_ctx** out) {
    if (!dir || !out) { g_dir_err = "null argument"; return GL3_E_ARG; }
    std::string text;
    if (!read_file(std::string(dir) + "/config.json", text)) { g_dir_err = std::string("cannot read ") + dir + "/config.json"; return GL3_E_ARG; }
    JVal cfg;
    if (!parse_json(text.data(), text.size(), cfg, g_dir_err)) return GL3_E_ARG;
    const JVal* arch = cfg.get("architecture");
    if (!arch || arch->kind != JVal::STR) { g_dir_err = "config: missing 'architecture'"; return GL3_E_ARG; }
    const Design* design = nullptr;
    for (const Design& d : DESIGNS)
        if (arch->str == d.architecture) design = &d;
    if (!design) { g_dir_err = "no model class is registered for architecture '" + arch->str + "'"; return GL3_E_UNSUPPORTED; }
    gl3_model_desc d{};
    d.struct_size = sizeof d;
    std::vector<gl3_layer_desc> layers;
    DescStore store;
    std::string err;
    if (!design->describe(cfg, d, layers, store, err)) { g_dir_err = err; return GL3_E_ARG; }
    d.layer_descs = layers.data();
    d.ctx = opts && opts->ctx > 0 ? opts->ctx : 4096;
    d.max_batch = opts && opts->max_batch > 0 ? opts->max_batch : 512;
    d.device = opts ? opts->device : 0;
    d.flags = opts ? opts->flags : 0;
    d.n_seqs = opts && opts->n_seqs > 0 ? opts->n_seqs : 1;
    d.tp_size = 1;

    // the weights
    const std::string wpath = std::string(dir) + "/model.safetensors";
    const int fd = open(wpath.c_str(), O_RDONLY);
    if (fd < 0) { g_dir_err = "cannot open " + wpath; return GL3_E_ARG; }
    struct stat st;
    Mapping map;
    if (fstat(fd, &st) == 0 && st.st_size >= 8) { map.n = (size_t)st.st_size; map.p = mmap(nullptr, map.n, PROT_READ, MAP_PRIVATE, fd, 0); }
    close(fd);
    if (map.p == MAP_FAILED) { g_dir_err = "cannot map " + wpath; return GL3_E_ARG; }
    const uint8_t* base = (const uint8_t*)map.p;
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | base[i];
    if (hlen > map.n - 8) { g_dir_err = "safetensors: header length exceeds the file"; return GL3_E_ARG; }
    JVal hdr;
    if (!parse_json((const char*)base + 8, (size_t)hlen, hdr, g_dir_err)) return GL3_E_ARG;
    if (hdr.kind != JVal::OBJ) { g_dir_err = "safetensors: header is not an object"; return GL3_E_ARG; }
    const uint8_t* data = base + 8 + hlen;
    const uint64_t data_n = map.n - 8 - hlen;

    gl3_ctx* ctx = nullptr;
    int32_t r = gl3_create(&d, &ctx);
    if (r != GL3_OK) { g_dir_err = gl3_last_error(nullptr); return r; }
    // parts of stacked tensors: (layer, id) -> expert -> (data, bytes, type)
    struct Part { const uint8_t* p; uint64_t n; int type; };
    std::map<std::pair<int32_t, int32_t>, std::map<int32_t, Part>> stacks;
    for (auto& kv : hdr.obj) {
        if (kv.first == "__metadata__") continue;
        int32_t id = 0, layer = 0, expert = -1;
        if (!design->tensor(kv.first, id, layer, expert)) continue;          // a name the design does not know carries nothing it computes with
        const JVal *dt = kv.second.get("dtype"), *shape = kv.second.get("shape"), *offs = kv.second.get("data_offsets");
        if (!dt || dt->kind != JVal::STR || !shape || shape->kind != JVal::ARR || !offs || offs->kind != JVal::ARR || offs->arr.size() != 2) {
            g_dir_err = "safetensors: malformed entry '" + kv.first + "'"; gl3_destroy(ctx); return GL3_E_ARG;
        }
        int type, es;
        if (dt->str == "BF16") { type = GL3_TYPE_BF16; es = 2; }
        else if (dt->str == "F32") { type = GL3_TYPE_F32; es = 4; }
        else { g_dir_err = "safetensors: tensor '" + kv.first + "' has dtype " + dt->str + " (BF16 or F32 expected)"; gl3_destroy(ctx); return GL3_E_UNSUPPORTED; }
        double count = 1;
        for (auto& s : shape->arr) count *= s.kind == JVal::NUM ? s.num : -1;
        const double a = offs->arr[0].num, b = offs->arr[1].num;
        if (!(count >= 0) || !(a >= 0) || !(b >= a) || b > (double)data_n || b - a != count * es) {
            g_dir_err = "safetensors: tensor '" + kv.first + "' has offsets that do not fit its shape or the file"; gl3_destroy(ctx); return GL3_E_ARG;
        }
        if (expert >= 0) { stacks[{layer, id}][expert] = Part{data + (uint64_t)a, (uint64_t)(b - a), type}; continue; }
        r = gl3_upload_tensor(ctx, id, layer, data + (uint64_t)a, (uint64_t)(b - a), type);
        if (r != GL3_OK) { g_dir_err = "tensor '" + kv.first + "': " + gl3_last_error(ctx); gl3_destroy(ctx); return r; }
    }
    for (auto& st : stacks) {
        const int32_t layer = st.first.first, id = st.first.second;
        const int want = layer >= 0 && layer < (int)layers.size() ? layers[layer].experts : 0;          // (a second mixer has no experts)
        const Part& first = st.second.begin()->second;
        bool ok = (int)st.second.size() == want && st.second.rbegin()->first == want - 1;
        for (auto& pt : st.second) ok = ok && pt.second.n == first.n && pt.second.type == first.type;
        if (!ok) { g_dir_err = "layer " + std::to_string(layer) + ": the experts' tensors do not match the router (count, size or type)"; gl3_destroy(ctx); return GL3_E_ARG; }
        std::vector<uint8_t> whole((size_t)first.n * want);
        for (auto& pt : st.second) memcpy(whole.data() + (size_t)pt.first * first.n, pt.second.p, (size_t)first.n);
        r = gl3_upload_tensor(ctx, id, layer, whole.data(), whole.size(), first.type);
        if (r != GL3_OK) { g_dir_err = "layer " + std::to_string(layer) + ", stacked experts: " + gl3_last_error(ctx); gl3_destroy(ctx); return r; }
    }
    r = gl3_finalize(ctx);
    if (r != GL3_OK) { g_dir_err = gl3_last_error(ctx); gl3_destroy(ctx); return r; }
    *out = ctx;
    return GL3_OK;
}

}  // extern "C"
