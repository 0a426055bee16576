// Checkpoint side of the path: the safetensors reader and weight naming of the reference's
// crates/llm/src/hf_weights.rs:65-159, the offline int8 quantiser of crates/llm/src/quantize.rs:28-42,
// 313-337 (file level; the per-channel rule itself is mynn_quantize_per_channel), and the upload of a
// Llama checkpoint into the `initializer` array that model_init takes (names as ModelSpec::from_hf,
// crates/llm/src/decoder.rs:570-660).  Host code only, except for the uploads.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "mynn_common.h"

namespace mynn {

// ---- a JSON reader just large enough for a safetensors header and model.safetensors.index.json ----
struct Json {
    enum Kind { NUL, NUM, STR, ARR, OBJ, BOOL } kind = NUL;
    double num = 0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;  // insertion order
    const Json *get(const char *key) const {
        for (auto &kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
};
struct JsonParser {
    const char *p, *end;  // [p, end) is followed by a NUL (parse_json copies the text), so strtod cannot run past it
    bool ok = true;
    int depth = 0;
    static constexpr int kMaxDepth = 32;  // a safetensors header nests 3 deep
    void ws() {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) p++;
    }
    bool eat(char c) {
        ws();
        if (p < end && *p == c) {
            p++;
            return true;
        }
        return false;
    }
    std::string string() {
        std::string s;
        if (!eat('"')) {
            ok = false;
            return s;
        }
        while (p < end && *p != '"') {
            if (*p == '\\' && p + 1 < end) {
                p++;
                switch (*p) {
                case 'n': s += '\n'; break;
                case 't': s += '\t'; break;
                case 'u':  // tensor names are ASCII; keep the escape verbatim
                    s += "\\u";
                    break;
                default: s += *p;
                }
                p++;
            } else s += *p++;
        }
        if (p >= end) ok = false;
        else p++;
        return s;
    }
    Json value() {
        Json j;
        ws();
        if (p >= end) {
            ok = false;
            return j;
        }
        if ((*p == '{' || *p == '[') && ++depth > kMaxDepth) {
            ok = false;
            return j;
        }
        if (*p == '{') {
            p++;
            j.kind = Json::OBJ;
            if (eat('}')) {
                depth--;
                return j;
            }
            do {
                std::string k = string();
                if (!ok || !eat(':')) {
                    ok = false;
                    return j;
                }
                j.obj.emplace_back(std::move(k), value());
                if (!ok) return j;
            } while (eat(','));
            if (!eat('}')) ok = false;
            depth--;
        } else if (*p == '[') {
            p++;
            j.kind = Json::ARR;
            if (eat(']')) {
                depth--;
                return j;
            }
            do {
                j.arr.push_back(value());
                if (!ok) return j;
            } while (eat(','));
            if (!eat(']')) ok = false;
            depth--;
        } else if (*p == '"') {
            j.kind = Json::STR;
            j.str = string();
        } else if ((end - p >= 4 && (!strncmp(p, "true", 4) || !strncmp(p, "null", 4))) || (end - p >= 5 && !strncmp(p, "false", 5))) {
            j.kind = *p == 'n' ? Json::NUL : Json::BOOL;
            j.num = *p == 't';
            p += *p == 'f' ? 5 : 4;
        } else {
            char *q = nullptr;
            j.kind = Json::NUM;
            j.num = strtod(p, &q);
            if (q == p || q > end) ok = false;
            p = q;
        }
        return j;
    }
};
static bool parse_json(const char *data, size_t n, Json &out) {
    const std::string text(data, n);  // NUL-terminated copy: the mapped header may end exactly at the end of the file
    JsonParser ps{text.c_str(), text.c_str() + n};
    out = ps.value();
    return ps.ok;
}

// a JSON number that must be a non-negative integer below 2^53 (offsets, extents): false otherwise
static bool as_size(const Json &j, size_t *out) {
    if (j.kind != Json::NUM || !(j.num >= 0.0) || j.num > 9007199254740992.0 || j.num != (double)(uint64_t)j.num) return false;
    *out = (size_t)j.num;
    return true;
}

// ---- shards ---------------------------------------------------------------------------------------
struct Shard {
    std::string path;
    void *map = nullptr;
    size_t bytes = 0;
    ~Shard() {
        if (map) munmap(map, bytes);
    }
};
struct Entry {
    const Shard *shard;
    size_t offset, length;
    int dtype;  // MYNN_F32 / MYNN_BF16 / MYNN_F16 / MYNN_I8
    std::vector<int64_t> shape;
};

}  // namespace mynn

struct mynn_weights {
    std::vector<std::unique_ptr<mynn::Shard>> shards;
    std::map<std::string, mynn::Entry> entries;
    std::vector<std::string> order;  // names in file order
};

namespace mynn {

static bool file_exists(const std::string &p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
static bool is_dir(const std::string &p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}
static int dtype_of(const std::string &s) {
    if (s == "F32") return MYNN_F32;
    if (s == "BF16") return MYNN_BF16;
    if (s == "F16") return MYNN_F16;
    if (s == "I8") return MYNN_I8;
    return -1;
}
static const char *dtype_name(int d) {
    return d == MYNN_F32 ? "F32" : d == MYNN_BF16 ? "BF16" : d == MYNN_F16 ? "F16" : "I8";
}
static size_t dtype_bytes(int d) { return d == MYNN_F32 ? 4 : d == MYNN_I8 ? 1 : 2; }

// hf_weights.rs:120-143: every tensor of the shard, offsets relative to the end of the header
static int add_shard(mynn_weights &w, const std::string &path) {
    int fd = open(path.c_str(), O_RDONLY);
    MYNN_REQUIRE(fd >= 0, MYNN_ERR_INVALID, "weights: cannot open %s", path.c_str());
    struct stat st;
    fstat(fd, &st);
    auto sh = std::make_unique<Shard>();
    sh->path = path;
    sh->bytes = (size_t)st.st_size;
    sh->map = sh->bytes ? mmap(nullptr, sh->bytes, PROT_READ, MAP_PRIVATE, fd, 0) : nullptr;
    close(fd);
    if (sh->map == MAP_FAILED) sh->map = nullptr;
    MYNN_REQUIRE(sh->map && sh->bytes >= 8, MYNN_ERR_INVALID, "weights: cannot map %s", path.c_str());
    uint64_t hlen;
    memcpy(&hlen, sh->map, 8);
    MYNN_REQUIRE(hlen <= sh->bytes - 8, MYNN_ERR_INVALID, "weights: %s: header length %llu exceeds the file", path.c_str(),
                 (unsigned long long)hlen);
    Json hdr;
    MYNN_REQUIRE(parse_json((const char *)sh->map + 8, (size_t)hlen, hdr) && hdr.kind == Json::OBJ, MYNN_ERR_INVALID,
                 "weights: %s: malformed header", path.c_str());
    const size_t data_start = 8 + (size_t)hlen;
    for (auto &kv : hdr.obj) {
        if (kv.first == "__metadata__") continue;
        const Json *dt = kv.second.get("dtype"), *shp = kv.second.get("shape"), *off = kv.second.get("data_offsets");
        MYNN_REQUIRE(dt && shp && off && off->arr.size() == 2, MYNN_ERR_INVALID, "weights: %s: malformed entry %s",
                     path.c_str(), kv.first.c_str());
        Entry e;
        e.shard = sh.get();
        e.dtype = dtype_of(dt->str);
        MYNN_REQUIRE(e.dtype >= 0, MYNN_ERR_UNSUPPORTED, "weights: %s: dtype %s of %s", path.c_str(), dt->str.c_str(),
                     kv.first.c_str());
        MYNN_REQUIRE(dt->kind == Json::STR && shp->kind == Json::ARR && off->kind == Json::ARR && shp->arr.size() <= 8, MYNN_ERR_INVALID,
                     "weights: %s: malformed entry %s", path.c_str(), kv.first.c_str());
        // every extent and offset is a checked unsigned integer; products and sums cannot wrap
        size_t count = 1, off0 = 0, off1 = 0;
        bool sane = as_size(off->arr[0], &off0) && as_size(off->arr[1], &off1) && off0 <= off1 && off1 <= sh->bytes - data_start;
        for (auto &d : shp->arr) {
            size_t ext = 0;
            sane = sane && as_size(d, &ext) && (ext == 0 || count <= sh->bytes / ext);  // (count * ext stays within the file size)
            if (!sane) break;
            count *= ext;
            e.shape.push_back((int64_t)ext);
        }
        MYNN_REQUIRE(sane && count <= (off1 - off0) && off1 - off0 == count * dtype_bytes(e.dtype), MYNN_ERR_INVALID,
                     "weights: %s: %s has inconsistent shape or offsets", path.c_str(), kv.first.c_str());
        e.offset = data_start + off0;
        e.length = off1 - off0;
        if (!w.entries.count(kv.first)) w.order.push_back(kv.first);
        w.entries[kv.first] = std::move(e);
    }
    w.shards.push_back(std::move(sh));
    return 0;
}

// model.safetensors.index.json: the distinct shard names of "weight_map", in order of first appearance
static int shards_of_index(const std::string &index_path, std::vector<std::string> &files) {
    FILE *f = fopen(index_path.c_str(), "rb");
    MYNN_REQUIRE(f, MYNN_ERR_INVALID, "weights: cannot open %s", index_path.c_str());
    std::string text;
    char buf[65536];
    size_t n;
    while ((n = fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, n);
    fclose(f);
    Json j;
    MYNN_REQUIRE(parse_json(text.data(), text.size(), j), MYNN_ERR_INVALID, "weights: %s: malformed json", index_path.c_str());
    const Json *wm = j.get("weight_map");
    MYNN_REQUIRE(wm && wm->kind == Json::OBJ, MYNN_ERR_INVALID, "weights: %s: missing weight_map", index_path.c_str());
    const std::string dir = index_path.substr(0, index_path.find_last_of('/') + 1);
    for (auto &kv : wm->obj) {
        const std::string &name = kv.second.str;
        MYNN_REQUIRE(kv.second.kind == Json::STR && !name.empty() && name.find('/') == std::string::npos &&
                         name.find('\\') == std::string::npos && name != "." && name != "..",
                     MYNN_ERR_INVALID, "weights: %s: shard name '%s' is not a plain file name", index_path.c_str(), name.c_str());
        std::string p = dir + name;
        bool seen = false;
        for (auto &s : files) seen |= s == p;
        if (!seen) files.push_back(p);
    }
    return 0;
}

// hf_weights.rs:75-91 for a directory; a file is read as one shard
static int source_files(const std::string &path, bool prefer_int8, std::vector<std::string> &files) {
    if (!is_dir(path)) {
        files.push_back(path);
        return 0;
    }
    const std::string dir = path.back() == '/' ? path : path + "/";
    if (prefer_int8 && file_exists(dir + "model.int8.safetensors")) files.push_back(dir + "model.int8.safetensors");
    else if (file_exists(dir + "model.safetensors.index.json")) return shards_of_index(dir + "model.safetensors.index.json", files);
    else if (file_exists(dir + "model.safetensors")) files.push_back(dir + "model.safetensors");
    else return fail(MYNN_ERR_INVALID, "weights: no safetensors in %s", path.c_str());
    return 0;
}

static float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

static void to_f32(const Entry &e, std::vector<float> &out) {
    const char *src = (const char *)e.shard->map + e.offset;
    const size_t n = e.length / dtype_bytes(e.dtype);
    out.resize(n);
    for (size_t i = 0; i < n; i++) {
        if (e.dtype == MYNN_F32) memcpy(&out[i], src + 4 * i, 4);
        else {
            uint16_t b;
            memcpy(&b, src + 2 * i, 2);
            out[i] = e.dtype == MYNN_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
        }
    }
}

// values of a float tensor in the storage type `dt` (16-bit types; RNE from f32)
static void to_storage(const Entry &e, int dt, std::vector<uint16_t> &out) {
    if (e.dtype == dt) {
        out.resize(e.length / 2);
        memcpy(out.data(), (const char *)e.shard->map + e.offset, e.length);
        return;
    }
    std::vector<float> f;
    to_f32(e, f);
    out.resize(f.size());
    for (size_t i = 0; i < f.size(); i++)
        out[i] = dt == MYNN_BF16 ? f32_to_bf16_bits(f[i]) : __builtin_bit_cast(uint16_t, (_Float16)f[i]);
}

static bool ends_with(const std::string &s, const char *suffix) {
    const size_t n = strlen(suffix);
    return s.size() >= n && !s.compare(s.size() - n, n, suffix);
}
// quantize.rs:28-42
static bool should_quantize(const std::string &name) {
    static const char *pat[] = {"q_proj.weight",  "k_proj.weight",    "v_proj.weight",  "o_proj.weight",      "gate_proj.weight",
                                "up_proj.weight", "down_proj.weight", "lm_head.weight", "embed_tokens.weight"};
    for (const char *p : pat)
        if (ends_with(name, p)) return true;
    return false;
}

struct OutTensor {
    std::string name;
    int dtype;
    std::vector<int64_t> shape;
    std::vector<char> data;
};
static int write_safetensors(const std::string &dst, const std::vector<OutTensor> &ts) {
    std::string hdr = "{";
    size_t off = 0;
    for (size_t i = 0; i < ts.size(); i++) {
        const OutTensor &t = ts[i];
        hdr += (i ? ",\"" : "\"") + t.name + "\":{\"dtype\":\"" + dtype_name(t.dtype) + "\",\"shape\":[";
        for (size_t d = 0; d < t.shape.size(); d++) hdr += (d ? "," : "") + std::to_string(t.shape[d]);
        hdr += "],\"data_offsets\":[" + std::to_string(off) + "," + std::to_string(off + t.data.size()) + "]}";
        off += t.data.size();
    }
    hdr += "}";
    while (hdr.size() % 8) hdr += ' ';
    FILE *f = fopen(dst.c_str(), "wb");
    MYNN_REQUIRE(f, MYNN_ERR_INVALID, "weights: cannot create %s", dst.c_str());
    const uint64_t hlen = hdr.size();
    bool ok = fwrite(&hlen, 8, 1, f) == 1 && fwrite(hdr.data(), 1, hdr.size(), f) == hdr.size();
    for (auto &t : ts) ok = ok && (t.data.empty() || fwrite(t.data.data(), 1, t.data.size(), f) == t.data.size());
    ok = fclose(f) == 0 && ok;
    MYNN_REQUIRE(ok, MYNN_ERR_INVALID, "weights: short write to %s", dst.c_str());
    return 0;
}

}  // namespace mynn

using namespace mynn;

static mynn_weights *weights_open_impl(const char *path) {
    if (!path) {
        set_error("weights_open: null path");
        return nullptr;
    }
    std::vector<std::string> files;
    if (source_files(path, true, files)) return nullptr;
    auto w = std::make_unique<mynn_weights>();
    for (auto &f : files)
        if (add_shard(*w, f)) return nullptr;
    return w.release();
}
extern "C" void mynn_weights_close(mynn_weights *w) { delete w; }
extern "C" int mynn_weights_count(const mynn_weights *w) { return w ? (int)w->order.size() : 0; }
extern "C" const char *mynn_weights_name(const mynn_weights *w, int i) {
    return w && i >= 0 && i < (int)w->order.size() ? w->order[i].c_str() : nullptr;
}
extern "C" int mynn_weights_find(const mynn_weights *w, const char *name, int *dtype, int64_t *shape, int *ndim,
                                 const void **data, size_t *nbytes) {
    MYNN_REQUIRE(w && name, MYNN_ERR_INVALID, "weights_find: null argument");
    auto it = w->entries.find(name);
    MYNN_REQUIRE(it != w->entries.end(), MYNN_ERR_INVALID, "weights: no tensor named %s", name);
    const Entry &e = it->second;
    if (dtype) *dtype = e.dtype;
    if (ndim) *ndim = (int)e.shape.size();
    if (shape)
        for (size_t i = 0; i < e.shape.size() && i < 8; i++) shape[i] = e.shape[i];
    if (data) *data = (const char *)e.shard->map + e.offset;
    if (nbytes) *nbytes = e.length;
    return 0;
}

// quantize.rs:313-337 (and copy_view :170-188: an f16 tensor that is not quantised is stored as bf16)
static int quantize_safetensors_int8_impl(const char *src, const char *dst, int *quantized, int *passthrough) {
    MYNN_REQUIRE(src && dst, MYNN_ERR_INVALID, "quantize_safetensors_int8: null path");
    std::vector<std::string> files;
    int rc = source_files(src, false, files);
    if (rc) return rc;
    mynn_weights w;
    for (auto &f : files)
        if ((rc = add_shard(w, f))) return rc;
    std::vector<OutTensor> out;
    int nq = 0, np = 0;
    for (auto &name : w.order) {
        const Entry &e = w.entries[name];
        if (should_quantize(name)) {
            MYNN_REQUIRE(e.shape.size() >= 2 && e.dtype != MYNN_I8, MYNN_ERR_INVALID,
                         "quantize_safetensors_int8: %s is not a float matrix", name.c_str());
            const size_t cols = (size_t)e.shape.back(), rows = e.length / dtype_bytes(e.dtype) / cols;
            std::vector<float> f;
            to_f32(e, f);
            OutTensor q{name, MYNN_I8, e.shape, std::vector<char>(rows * cols)};
            OutTensor s{name + ".scale", MYNN_BF16, {(int64_t)rows}, std::vector<char>(rows * 2)};
            rc = mynn_quantize_per_channel((int8_t *)q.data.data(), s.data.data(), f.data(), rows, cols, MYNN_BF16);
            if (rc) return rc;
            out.push_back(std::move(q));
            out.push_back(std::move(s));
            nq++;
        } else {
            OutTensor t{name, e.dtype, e.shape, {}};
            if (e.dtype == MYNN_F16) {
                std::vector<uint16_t> b;
                to_storage(e, MYNN_BF16, b);
                t.dtype = MYNN_BF16;
                t.data.assign((const char *)b.data(), (const char *)b.data() + b.size() * 2);
            } else {
                const char *p = (const char *)e.shard->map + e.offset;
                t.data.assign(p, p + e.length);
            }
            out.push_back(std::move(t));
            np++;
        }
    }
    if (quantized) *quantized = nq;
    if (passthrough) *passthrough = np;
    return write_safetensors(dst, out);
}

// ---- upload: the `initializer` array of model_init from a checkpoint --------------------------------
struct mynn_device_weights {
    std::vector<void *> init;    // 4 + 16 * n_layers entries, device pointers (nullptr scale slots when dense)
    std::vector<void *> owned;   // every allocation
    int weights_int8 = 0;
};

static int upload(mynn_device_weights &dw, const void *host, size_t bytes, void **out) {
    void *d = nullptr;
    MYNN_HIP(hipMalloc(&d, bytes ? bytes : 1));
    dw.owned.push_back(d);
    MYNN_HIP(hipMemcpy(d, host, bytes, hipMemcpyHostToDevice));
    *out = d;
    return 0;
}
// a float tensor in cfg.dtype
static int upload_float(mynn_device_weights &dw, const mynn_weights &w, const std::string &name, int dt, size_t want_elems) {
    auto it = w.entries.find(name);
    MYNN_REQUIRE(it != w.entries.end(), MYNN_ERR_INVALID, "weights: no tensor named %s", name.c_str());
    MYNN_REQUIRE(it->second.dtype != MYNN_I8, MYNN_ERR_INVALID, "weights: %s is int8, a float tensor was expected", name.c_str());
    std::vector<uint16_t> b;
    to_storage(it->second, dt, b);
    MYNN_REQUIRE(b.size() == want_elems, MYNN_ERR_INVALID, "weights: %s has %zu elements, the config needs %zu", name.c_str(),
                 b.size(), want_elems);
    void *d;
    int rc = upload(dw, b.data(), b.size() * 2, &d);
    if (rc) return rc;
    dw.init.push_back(d);
    return 0;
}
// a linear weight: int8 + "<name>.scale" (hf_weights.rs:153-158), or a float matrix and an empty scale slot
static int upload_linear(mynn_device_weights &dw, const mynn_weights &w, const std::string &name, int dt, size_t N, size_t K) {
    auto it = w.entries.find(name);
    MYNN_REQUIRE(it != w.entries.end(), MYNN_ERR_INVALID, "weights: no tensor named %s", name.c_str());
    const Entry &e = it->second;
    MYNN_REQUIRE((e.dtype == MYNN_I8) == (dw.weights_int8 != 0), MYNN_ERR_INVALID,
                 "weights: %s: int8 and float linear weights are mixed in one checkpoint", name.c_str());
    if (e.dtype != MYNN_I8) {
        int rc = upload_float(dw, w, name, dt, N * K);
        if (rc) return rc;
        dw.init.push_back(nullptr);
        return 0;
    }
    MYNN_REQUIRE(e.length == N * K, MYNN_ERR_INVALID, "weights: %s has %zu elements, the config needs %zu", name.c_str(),
                 e.length, N * K);
    void *d;
    int rc = upload(dw, (const char *)e.shard->map + e.offset, e.length, &d);
    if (rc) return rc;
    dw.init.push_back(d);
    return upload_float(dw, w, name + ".scale", dt, N);
}

static mynn_device_weights *weights_upload_impl(const mynn_weights *w, const mynn_model_config *c) {
    if (!w || !c) {
        set_error("weights_upload: null argument");
        return nullptr;
    }
    auto e = w->entries.find("model.embed_tokens.weight");
    if (e == w->entries.end()) {
        set_error("weights: no tensor named model.embed_tokens.weight");
        return nullptr;
    }
    auto dw = std::make_unique<mynn_device_weights>();
    dw->weights_int8 = e->second.dtype == MYNN_I8;
    const int dt = c->dtype;
    const size_t H = c->hidden, QD = (size_t)c->n_heads * c->head_dim, KD = (size_t)c->n_kv_heads * c->head_dim, F = c->ffn,
                 V = c->vocab;
    auto fail_free = [&](int) {
        for (void *p : dw->owned) (void)hipFree(p);
        return (mynn_device_weights *)nullptr;
    };
    int rc = upload_linear(*dw, *w, "model.embed_tokens.weight", dt, V, H);
    for (int l = 0; l < c->n_layers && !rc; l++) {
        const std::string p = "model.layers." + std::to_string(l);
        rc = upload_float(*dw, *w, p + ".input_layernorm.weight", dt, H);
        // (qkv_bias: `{base}.bias` behind each of the three, ModelSpec::from_hf, decoder.rs:557-569)
        if (!rc) rc = upload_linear(*dw, *w, p + ".self_attn.q_proj.weight", dt, QD, H);
        if (!rc && c->qkv_bias) rc = upload_float(*dw, *w, p + ".self_attn.q_proj.bias", dt, QD);
        if (!rc) rc = upload_linear(*dw, *w, p + ".self_attn.k_proj.weight", dt, KD, H);
        if (!rc && c->qkv_bias) rc = upload_float(*dw, *w, p + ".self_attn.k_proj.bias", dt, KD);
        if (!rc) rc = upload_linear(*dw, *w, p + ".self_attn.v_proj.weight", dt, KD, H);
        if (!rc && c->qkv_bias) rc = upload_float(*dw, *w, p + ".self_attn.v_proj.bias", dt, KD);
        if (!rc) rc = upload_linear(*dw, *w, p + ".self_attn.o_proj.weight", dt, H, QD);
        if (!rc) rc = upload_float(*dw, *w, p + ".post_attention_layernorm.weight", dt, H);
        if (!rc) rc = upload_linear(*dw, *w, p + ".mlp.gate_proj.weight", dt, F, H);
        if (!rc) rc = upload_linear(*dw, *w, p + ".mlp.up_proj.weight", dt, F, H);
        if (!rc) rc = upload_linear(*dw, *w, p + ".mlp.down_proj.weight", dt, H, F);
    }
    if (!rc) rc = upload_float(*dw, *w, "model.norm.weight", dt, H);
    if (!rc) rc = upload_linear(*dw, *w, "lm_head.weight", dt, V, H);
    if (rc) return fail_free(rc);
    return dw.release();
}
extern "C" void **mynn_device_weights_initializer(mynn_device_weights *dw) { return dw ? dw->init.data() : nullptr; }
extern "C" int mynn_device_weights_int8(const mynn_device_weights *dw) { return dw ? dw->weights_int8 : 0; }
extern "C" void mynn_device_weights_free(mynn_device_weights *dw) {
    if (!dw) return;
    for (void *p : dw->owned) (void)hipFree(p);
    delete dw;
}

// No exception crosses the C boundary: an allocation that fails (a corrupt header can ask for one) becomes an error.
template <typename R, typename F>
static R guarded(F &&f, R on_fail) {
    try {
        return f();
    } catch (const std::exception &e) {
        set_error("weights: %s", e.what());
    } catch (...) {
        set_error("weights: unknown failure");
    }
    return on_fail;
}
extern "C" mynn_weights *mynn_weights_open(const char *path) {
    return guarded<mynn_weights *>([&] { return weights_open_impl(path); }, nullptr);
}
extern "C" int mynn_quantize_safetensors_int8(const char *src, const char *dst, int *quantized, int *passthrough) {
    return guarded<int>([&] { return quantize_safetensors_int8_impl(src, dst, quantized, passthrough); }, (int)MYNN_ERR_INVALID);
}
extern "C" mynn_device_weights *mynn_weights_upload(const mynn_weights *w, const mynn_model_config *c) {
    return guarded<mynn_device_weights *>([&] { return weights_upload_impl(w, c); }, nullptr);
}
