// GGUF intake (host code only): the header parser of crates/repack/src/gguf_header/parser.rs:124-239,
// the llama-family tensor names of crates/repack/src/gguf_names/llama.rs:14-60, and the one
// source convention a llama GGUF needs, the rotary row un-permutation of
// crates/repack/src/gguf_checkpoint/conventions.rs:133-243.  The file is mapped read-only; tensor
// bytes are handed to tsv_open where they lie (GGUF block layouts are the install's own), and the
// mapping is dropped once tsv_open has re-tiled them into device memory.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <climits>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <string>
#include <vector>

#include "tsv_internal.h"

using tsv::set_error;

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;  // "GGUF", little endian (gguf_header/types.rs:6)
constexpr uint32_t GGUF_VERSION = 3;          // types.rs:19: v1 / v2 differ in field widths
constexpr uint64_t DEFAULT_ALIGNMENT = 32;    // types.rs:15
constexpr uint32_t MAX_ARRAY_DEPTH = 64;      // types.rs:26
constexpr uint64_t KEPT_ARRAY = 1 << 16;      // numeric arrays up to this length are kept as values

struct Value {
    enum Kind { NONE, UINT, INT, FLOAT, BOOL, STRING, ARRAY } kind = NONE;
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0.0;
    std::string s;
    uint64_t count = 0;          // ARRAY: number of elements
    std::vector<double> items;   // ARRAY of numbers, when short enough to keep
};

struct TensorInfo {
    uint32_t type = 0;
    std::vector<uint64_t> dims;  // ggml order: dims[0] is the row length
    uint64_t offset = 0;         // relative to the data region
};

}  // namespace

struct tsv_gguf {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t size = 0;
    uint64_t alignment = DEFAULT_ALIGNMENT, data_start = 0;
    std::map<std::string, Value> meta;
    std::map<std::string, TensorInfo> tensors;
    ~tsv_gguf() {
        if (map) munmap((void*)map, size);
        if (fd >= 0) close(fd);
    }
};

namespace {

// Bounds-checked forward reader (parser.rs:10-41): a read that runs off the end fails by offset.
struct Cursor {
    const uint8_t* data;
    size_t size, pos = 0;
    bool ok = true;
    std::string why;

    const uint8_t* take(size_t n) {
        if (!ok) return nullptr;
        if (n > size - pos) {
            ok = false;
            why = "file too short: the header wants byte " + std::to_string((unsigned long long)pos + n);
            return nullptr;
        }
        const uint8_t* p = data + pos;
        pos += n;
        return p;
    }
    template <typename T>
    T num() {
        T v{};
        if (const uint8_t* p = take(sizeof(T))) std::memcpy(&v, p, sizeof(T));
        return v;
    }
    std::string str() {
        const uint64_t len = num<uint64_t>();
        if (!ok) return {};
        if (len > size - pos) {
            ok = false;
            why = "file too short: a string of " + std::to_string((unsigned long long)len) + " bytes runs past the end";
            return {};
        }
        const uint8_t* p = take((size_t)len);
        return p ? std::string((const char*)p, (size_t)len) : std::string();
    }
    void fail(const std::string& w) {
        if (ok) {
            ok = false;
            why = w;
        }
    }
};

// parser.rs:70-118: one metadata value; `depth` counts the enclosing arrays.
Value read_value(Cursor& c, uint32_t type, const std::string& key, uint32_t depth) {
    Value v;
    switch (type) {
        case 0: v.kind = Value::UINT; v.u = c.num<uint8_t>(); break;
        case 1: v.kind = Value::INT; v.i = c.num<int8_t>(); break;
        case 2: v.kind = Value::UINT; v.u = c.num<uint16_t>(); break;
        case 3: v.kind = Value::INT; v.i = c.num<int16_t>(); break;
        case 4: v.kind = Value::UINT; v.u = c.num<uint32_t>(); break;
        case 5: v.kind = Value::INT; v.i = c.num<int32_t>(); break;
        case 6: v.kind = Value::FLOAT; v.f = c.num<float>(); break;
        case 7: v.kind = Value::BOOL; v.u = c.num<uint8_t>() != 0; break;  // anything non-zero is true
        case 8: v.kind = Value::STRING; v.s = c.str(); break;
        case 9: {
            if (depth >= MAX_ARRAY_DEPTH) {
                c.fail("metadata key '" + key + "': arrays nested deeper than 64");
                break;
            }
            const uint32_t et = c.num<uint32_t>();
            const uint64_t len = c.num<uint64_t>();
            if (!c.ok) break;
            if (len > c.size) {  // the shortest element is one byte
                c.fail("metadata key '" + key + "': an array longer than the file");
                break;
            }
            v.kind = Value::ARRAY;
            v.count = len;
            const bool keep = len <= KEPT_ARRAY && et != 8 && et != 9;
            for (uint64_t k = 0; k < len && c.ok; k++) {
                Value e = read_value(c, et, key, depth + 1);
                if (keep) v.items.push_back(e.kind == Value::FLOAT ? e.f : e.kind == Value::INT ? (double)e.i : (double)e.u);
            }
            break;
        }
        case 10: v.kind = Value::UINT; v.u = c.num<uint64_t>(); break;
        case 11: v.kind = Value::INT; v.i = c.num<int64_t>(); break;
        case 12: v.kind = Value::FLOAT; v.f = c.num<double>(); break;
        default: c.fail("metadata key '" + key + "': value type " + std::to_string(type) + " is not a GGUF type");
    }
    return v;
}

// parse_header (parser.rs:124-239)
bool parse(tsv_gguf& g, std::string& why) {
    Cursor c{g.map, g.size};
    const uint32_t magic = c.num<uint32_t>();
    if (c.ok && magic != GGUF_MAGIC) c.fail("not a GGUF file: bad magic");
    const uint32_t version = c.num<uint32_t>();
    if (c.ok && version != GGUF_VERSION) c.fail("GGUF version " + std::to_string(version) + " is not supported (only 3)");
    const uint64_t n_tensors = c.num<uint64_t>(), n_kv = c.num<uint64_t>();
    // the smallest tensor entry is 32 bytes and the smallest key/value pair 13
    if (c.ok && (n_tensors > g.size / 32 || n_kv > g.size / 13)) c.fail("corrupt header: counts larger than the file can hold");
    for (uint64_t k = 0; k < n_kv && c.ok; k++) {
        const std::string key = c.str();
        const uint32_t type = c.num<uint32_t>();
        if (!c.ok) break;
        Value v = read_value(c, type, key, 0);
        if (c.ok && !g.meta.emplace(key, std::move(v)).second) c.fail("duplicate metadata key '" + key + "'");
    }
    for (uint64_t t = 0; t < n_tensors && c.ok; t++) {
        const std::string name = c.str();
        const uint32_t nd = c.num<uint32_t>();
        if (!c.ok) break;
        if (nd == 0 || nd > 4) {  // ggml's hard limit is four; zero dims is not a tensor
            c.fail("tensor '" + name + "': " + std::to_string(nd) + " dimensions");
            break;
        }
        TensorInfo info;
        for (uint32_t d = 0; d < nd && c.ok; d++) {
            const uint64_t dim = c.num<uint64_t>();
            if (c.ok && dim == 0) c.fail("tensor '" + name + "': a zero dimension");
            info.dims.push_back(dim);
        }
        info.type = c.num<uint32_t>();
        info.offset = c.num<uint64_t>();
        if (c.ok && !g.tensors.emplace(name, std::move(info)).second) c.fail("duplicate tensor '" + name + "'");
    }
    if (c.ok) {
        auto it = g.meta.find("general.alignment");
        if (it != g.meta.end()) {
            const Value& a = it->second;
            g.alignment = a.kind == Value::UINT ? a.u : a.kind == Value::INT && a.i > 0 ? (uint64_t)a.i : 0;
        }
        if (g.alignment == 0 || (g.alignment & (g.alignment - 1))) c.fail("general.alignment is not a power of two");
    }
    if (c.ok)
        for (const auto& kv : g.tensors)
            if (kv.second.offset % g.alignment) {
                c.fail("tensor '" + kv.first + "': offset is not a multiple of the file's alignment");
                break;
            }
    if (!c.ok) {
        why = c.why;
        return false;
    }
    g.data_start = (c.pos + g.alignment - 1) / g.alignment * g.alignment;
    return true;
}

// A tensor as rows of `cols` elements (every dimension but the first folded into the rows: the
// stacked experts of a 3-D tensor are then expert-major row runs), bounds-checked against the file.
int tensor_view(const tsv_gguf& g, const std::string& name, tsv_tensor* out) {
    auto it = g.tensors.find(name);
    if (it == g.tensors.end()) {
        set_error("gguf: no tensor '" + name + "'");
        return TSV_ERR_INVALID;
    }
    const TensorInfo& t = it->second;
    uint64_t rows = 1;
    for (size_t d = 1; d < t.dims.size(); d++) {
        if (t.dims[d] > (1ull << 40) / rows) {
            set_error("gguf: tensor '" + name + "': dimensions overflow");
            return TSV_ERR_INVALID;
        }
        rows *= t.dims[d];
    }
    // a row longer than any matmul's K cannot be a real tensor; past 2^31 the element count would
    // also wrap the signed arithmetic of the row-size helper
    if (t.dims[0] == 0 || t.dims[0] > (uint64_t)INT32_MAX) {
        set_error("gguf: tensor '" + name + "': first dimension outside 1..2^31-1");
        return TSV_ERR_INVALID;
    }
    const int64_t rb = tsv_row_bytes((int32_t)t.type, (int64_t)t.dims[0]);
    if (rb <= 0) {
        set_error("gguf: tensor '" + name + "': ggml type " + std::to_string(t.type) + " with rows of " +
                  std::to_string((unsigned long long)t.dims[0]) + " has no kernel here");
        return TSV_ERR_UNSUPPORTED;
    }
    // no product before the bound is known: rows * rb must fit what is left of the file
    const uint64_t begin = g.data_start + t.offset;
    if (begin < g.data_start || begin > g.size || rows > (g.size - begin) / (uint64_t)rb) {
        set_error("gguf: tensor '" + name + "' runs past the end of the file");
        return TSV_ERR_INVALID;
    }
    out->data = g.map + begin;
    out->dtype = (int32_t)t.type;
    out->rows = (int64_t)rows;
    out->cols = (int64_t)t.dims[0];
    return TSV_OK;
}

const Value* meta(const tsv_gguf& g, const std::string& key) {
    auto it = g.meta.find(key);
    return it == g.meta.end() ? nullptr : &it->second;
}

bool meta_number(const tsv_gguf& g, const std::string& key, double* out) {
    const Value* v = meta(g, key);
    if (!v) return false;
    switch (v->kind) {
        case Value::UINT: case Value::BOOL: *out = (double)v->u; return true;
        case Value::INT: *out = (double)v->i; return true;
        case Value::FLOAT: *out = v->f; return true;
        default: return false;
    }
}

// conventions.rs:133-150: llama.cpp's converter reshapes each head's q / k rows from (2, D/2) to
// (D/2, 2) so that ggml's adjacent-pair rotation works; install row i of a head is GGUF row
// (i % (D/2)) * 2 + i / (D/2).  Rows are contiguous byte runs in every block layout, so this
// moves bytes without decoding any.  V never goes through the rotation and is not touched.
int unpermute_rotary_rows(const std::string& name, const tsv_tensor& src, int head_dim, std::vector<uint8_t>& dst) {
    if (head_dim <= 0 || head_dim % 2 || src.rows <= 0 || src.rows % head_dim) {
        set_error("gguf: tensor '" + name + "': " + std::to_string((long long)src.rows) + " rows do not split into whole heads of " +
                  std::to_string(head_dim));
        return TSV_ERR_INVALID;
    }
    const size_t rb = (size_t)tsv_row_bytes(src.dtype, src.cols), half = (size_t)head_dim / 2;
    dst.resize((size_t)src.rows * rb);
    const uint8_t* s = (const uint8_t*)src.data;
    for (size_t h0 = 0; h0 < (size_t)src.rows; h0 += (size_t)head_dim)
        for (size_t i = 0; i < (size_t)head_dim; i++)
            std::memcpy(dst.data() + (h0 + i) * rb, s + (h0 + (i % half) * 2 + i / half) * rb, rb);
    return TSV_OK;
}

}  // namespace

extern "C" int32_t tsv_gguf_open(const char* path, tsv_gguf** out) {
    if (!path || !out) {
        set_error("gguf_open: null path or output");
        return TSV_ERR_INVALID;
    }
    *out = nullptr;
    std::unique_ptr<tsv_gguf> g(new (std::nothrow) tsv_gguf());
    if (!g) {
        set_error("gguf_open: out of memory");
        return TSV_ERR_INVALID;
    }
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st {};
    if (g->fd < 0 || fstat(g->fd, &st) != 0 || st.st_size < 24) {
        set_error(std::string("gguf_open: cannot read '") + path + "' (missing, or shorter than a GGUF header)");
        return TSV_ERR_INVALID;
    }
    g->size = (size_t)st.st_size;
    void* m = mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) {
        set_error(std::string("gguf_open: cannot map '") + path + "'");
        return TSV_ERR_INVALID;
    }
    g->map = (const uint8_t*)m;
    std::string why;
    if (!parse(*g, why)) {
        set_error("gguf_open: " + why);
        return TSV_ERR_INVALID;
    }
    *out = g.release();
    return TSV_OK;
}

extern "C" void tsv_gguf_close(tsv_gguf* g) { delete g; }

extern "C" int64_t tsv_gguf_tensor_count(const tsv_gguf* g) { return g ? (int64_t)g->tensors.size() : -1; }

extern "C" int64_t tsv_gguf_data_start(const tsv_gguf* g) { return g ? (int64_t)g->data_start : -1; }

extern "C" int32_t tsv_gguf_tensor(const tsv_gguf* g, const char* name, tsv_tensor* out) {
    if (!g || !name || !out) {
        set_error("gguf_tensor: null argument");
        return TSV_ERR_INVALID;
    }
    return tensor_view(*g, name, out);
}

extern "C" int32_t tsv_gguf_meta_number(const tsv_gguf* g, const char* key, double* out) {
    if (!g || !key || !out) {
        set_error("gguf_meta_number: null argument");
        return TSV_ERR_INVALID;
    }
    if (!meta_number(*g, key, out)) {
        set_error(std::string("gguf: no numeric metadata '") + key + "'");
        return TSV_ERR_INVALID;
    }
    return TSV_OK;
}

extern "C" int32_t tsv_gguf_meta_string(const tsv_gguf* g, const char* key, char* buf, int32_t cap) {
    if (!g || !key || !buf || cap < 1) {
        set_error("gguf_meta_string: null argument");
        return TSV_ERR_INVALID;
    }
    const Value* v = meta(*g, key);
    if (!v || v->kind != Value::STRING) {
        set_error(std::string("gguf: no string metadata '") + key + "'");
        return TSV_ERR_INVALID;
    }
    const size_t n = std::min<size_t>(v->s.size(), (size_t)cap - 1);
    std::memcpy(buf, v->s.data(), n);
    buf[n] = 0;
    return TSV_OK;
}

// Opens a dense or routed-expert llama-family GGUF as a verify target: `llama` (q / k rows
// un-permuted), `qwen2` (q / k / v biases), `qwen3` and `qwen3moe` (per-head q / k norms),
// `gpt-oss` (biases, sinks, alternating window, YaRN, clamped SwiGLU).
extern "C" int32_t tsv_open_gguf(const char* path, int32_t max_context, tsv_ctx** out) {
    if (!out) {
        set_error("open_gguf: null output");
        return TSV_ERR_INVALID;
    }
    *out = nullptr;
    tsv_gguf* raw = nullptr;
    int rc = tsv_gguf_open(path, &raw);
    if (rc) return rc;
    std::unique_ptr<tsv_gguf> g(raw);

    const Value* av = meta(*g, "general.architecture");
    if (!av || av->kind != Value::STRING) {
        set_error("open_gguf: the file names no general.architecture");
        return TSV_ERR_INVALID;
    }
    const std::string arch = av->s;
    const bool is_llama = arch == "llama", is_qwen2 = arch == "qwen2", is_qwen3 = arch == "qwen3" || arch == "qwen3moe";
    const bool is_oss = arch == "gpt-oss";
    if (!is_llama && !is_qwen2 && !is_qwen3 && !is_oss) {
        set_error("open_gguf: architecture '" + arch + "' is not one this intake maps (llama, qwen2, qwen3, qwen3moe, gpt-oss)");
        return TSV_ERR_UNSUPPORTED;
    }
    auto need = [&](const char* suffix, double* v) {
        if (meta_number(*g, arch + "." + suffix, v)) return true;
        set_error("open_gguf: metadata '" + arch + "." + suffix + "' is missing");
        return false;
    };
    auto opt = [&](const char* suffix, double dflt) {
        double v;
        return meta_number(*g, arch + "." + suffix, &v) ? v : dflt;
    };
    double n_layers, hidden, n_heads, ffn = 0;
    if (!need("block_count", &n_layers) || !need("embedding_length", &hidden) || !need("attention.head_count", &n_heads))
        return TSV_ERR_INVALID;
    const double n_experts = opt("expert_count", 0);
    if (n_experts > 0) {
        ffn = opt("expert_feed_forward_length", 0);
        if (ffn <= 0 && !need("feed_forward_length", &ffn)) return TSV_ERR_INVALID;
    } else if (!need("feed_forward_length", &ffn)) {
        return TSV_ERR_INVALID;
    }
    const double kv_heads = opt("attention.head_count_kv", n_heads), key_len = opt("attention.key_length", hidden / n_heads);
    auto sane = [](double v, double hi) { return v >= 1 && v <= hi && v == (double)(int64_t)v; };
    if (!sane(n_layers, 4096) || !sane(hidden, 1 << 20) || !sane(n_heads, 1 << 16) || !sane(ffn, 1 << 24) ||
        !sane(kv_heads, 1 << 16) || !sane(key_len, 1024) || (n_experts != 0 && !sane(n_experts, 1 << 16))) {
        set_error("open_gguf: the model sizes in the metadata are not usable (layers, widths, head counts, experts)");
        return TSV_ERR_INVALID;
    }
    // a context-extension scheme this intake cannot express must refuse, not load a model that is
    // only wrong at long context
    bool yarn = false;
    if (const Value* st = meta(*g, arch + ".rope.scaling.type"))
        if (st->kind == Value::STRING && st->s != "none" && !st->s.empty()) {
            yarn = is_oss && st->s == "yarn";
            if (!yarn) {
                set_error("open_gguf: rope scaling '" + st->s + "' is not mapped");
                return TSV_ERR_UNSUPPORTED;
            }
        }

    tsv_model_desc d{};
    d.n_layers = (int32_t)n_layers;
    d.hidden = (int32_t)hidden;
    d.n_q_heads = (int32_t)n_heads;
    d.n_kv_heads = (int32_t)kv_heads;
    d.head_dim = (int32_t)key_len;
    d.ffn = (int32_t)ffn;
    d.rms_eps = (float)opt("attention.layer_norm_rms_epsilon", 1e-5);
    d.rope_theta = (float)opt("rope.freq_base", 10000.0);
    const double trained = opt("context_length", 0);
    d.max_context = max_context > 0 ? max_context : (int32_t)std::min(trained, 1048576.0);
    if (d.max_context < 1) {
        set_error("open_gguf: no context length given and none in the metadata");
        return TSV_ERR_INVALID;
    }
    if (opt("rope.dimension_count", d.head_dim) != d.head_dim) {
        set_error("open_gguf: partial rotation (rope.dimension_count below the head width) is not mapped");
        return TSV_ERR_UNSUPPORTED;
    }

    // gpt-oss: YaRN frequency table and magnitude scale (crates/repack/src/gguf_config/mod.rs:396-440:
    // factor and original context are required once the type says yarn, the betas default to
    // llama.cpp's 32 and 1), the clamped SwiGLU's constants (crates/gpu/src/shaders/moe_gguf.metal:528-556),
    // and a sliding window on EVEN layers (crates/runtime/src/families/gptoss/attn.rs:20-23).
    std::vector<float> yarn_freqs;
    double window = 0;
    if (is_oss) {
        if (yarn) {
            double factor, octx;
            if (!need("rope.scaling.factor", &factor) || !need("rope.scaling.original_context_length", &octx)) return TSV_ERR_INVALID;
            if (factor <= 0) {
                set_error("open_gguf: yarn factor is not usable");
                return TSV_ERR_INVALID;
            }
            if (meta(*g, arch + ".rope.scaling.yarn_log_multiplier")) {
                set_error("open_gguf: a yarn_log_multiplier other than the plain one is not mapped");
                return TSV_ERR_UNSUPPORTED;
            }
            yarn_freqs.resize((size_t)d.head_dim / 2);
            if ((rc = tsv_yarn_frequencies(d.head_dim, d.rope_theta, (float)factor, (int64_t)octx,
                                           (float)opt("rope.scaling.yarn_beta_fast", 32.0),
                                           (float)opt("rope.scaling.yarn_beta_slow", 1.0), yarn_freqs.data(), &d.rope_mscale)))
                return rc;
            d.rope_freqs = yarn_freqs.data();
        }
        d.act_alpha = 1.702f;
        d.act_limit = 7.0f;
        if (!need("attention.sliding_window", &window)) return TSV_ERR_INVALID;
        if (!sane(window, 1 << 30)) {
            set_error("open_gguf: attention.sliding_window is not usable");
            return TSV_ERR_INVALID;
        }
    }

    std::vector<std::vector<uint8_t>> owned;  // un-permuted q / k rows
    auto get = [&](const std::string& name, tsv_tensor* t, bool required) -> int {
        if (!g->tensors.count(name)) {
            if (!required) return TSV_OK;
            set_error("open_gguf: tensor '" + name + "' is missing");
            return TSV_ERR_INVALID;
        }
        return tensor_view(*g, name, t);
    };
    if ((rc = get("token_embd.weight", &d.embed, true))) return rc;
    if ((rc = get("output_norm.weight", &d.final_norm, true))) return rc;
    if ((rc = get("output.weight", &d.lm_head, false))) return rc;  // absent: tied to the embedding
    d.vocab = (int32_t)d.embed.rows;
    tsv_tensor factors{};
    if ((rc = get("rope_freqs.weight", &factors, false))) return rc;
    if (factors.data) {
        // llama-3's per-pair divisors (crates/compute/src/rope.rs:390-439), as llama.cpp stores them
        if (factors.dtype != 0 || factors.rows * factors.cols != d.head_dim / 2) {
            set_error("open_gguf: rope_freqs.weight is not head_dim / 2 f32 values");
            return TSV_ERR_INVALID;
        }
        d.rope_factors = (const float*)factors.data;
    }

    std::vector<tsv_layer> layers((size_t)d.n_layers);
    for (int l = 0; l < d.n_layers; l++) {
        tsv_layer& L = layers[(size_t)l];
        std::memset(&L, 0, sizeof L);
        const std::string p = "blk." + std::to_string(l) + ".";
        struct Slot {
            const char* suffix;
            tsv_tensor* t;
            bool required;
        };
        const bool routed = n_experts > 0;
        const Slot slots[] = {
            {"attn_norm.weight", &L.attn_norm, true}, {"attn_q.weight", &L.wq, true}, {"attn_k.weight", &L.wk, true},
            {"attn_v.weight", &L.wv, true}, {"attn_output.weight", &L.wo, true},
            // the pre-FFN norm (HF: post_attention_layernorm); gpt-oss files spell it post_attention_norm
            {is_oss ? "post_attention_norm.weight" : "ffn_norm.weight", &L.ffn_norm, true},
            {"attn_q_norm.weight", &L.q_norm, is_qwen3}, {"attn_k_norm.weight", &L.k_norm, is_qwen3},
            {"attn_q.bias", &L.bq, is_qwen2 || is_oss}, {"attn_k.bias", &L.bk, is_qwen2 || is_oss},
            {"attn_v.bias", &L.bv, is_qwen2 || is_oss},
            // gpt-oss (crates/repack/src/gguf_names/gpt_oss.rs:30-72): every projection and the router
            // carry a bias, one sink logit per q head, per-expert biases
            {"attn_output.bias", &L.bo, is_oss}, {"attn_sinks.weight", &L.sinks, is_oss},
            {"ffn_gate_inp.bias", &L.router_bias, is_oss}, {"ffn_gate_exps.bias", &L.be_gate, is_oss},
            {"ffn_up_exps.bias", &L.be_up, is_oss}, {"ffn_down_exps.bias", &L.be_down, is_oss},
            {"ffn_gate.weight", &L.w_gate, !routed}, {"ffn_up.weight", &L.w_up, !routed}, {"ffn_down.weight", &L.w_down, !routed},
            {"ffn_gate_inp.weight", &L.router, routed}, {"ffn_gate_exps.weight", &L.we_gate, routed},
            {"ffn_up_exps.weight", &L.we_up, routed}, {"ffn_down_exps.weight", &L.we_down, routed},
        };
        for (const Slot& s : slots) {
            // a slot another family owns is not read even when a file carries the name
            if (!s.required) continue;
            if ((rc = get(p + s.suffix, s.t, s.required))) return rc;
        }
        if (is_oss && l % 2 == 0) {
            L.window = (int32_t)window;
            // the reference's fp16 ring for windowed layers is a session option there too
            // (kv_cache.rs:122-131 fp16_ring_enabled); here the process environment asks for it
            const char* ring = getenv("TSV_KV_RING");
            L.ring = ring && ring[0] == '1';
        }
        if (routed) {
            L.n_experts = (int32_t)n_experts;
            const double used = opt("expert_used_count", 0);
            L.top_k = used >= 1 && used <= n_experts ? (int32_t)used : 0;  // 0 is refused by tsv_open
        }
        if (is_llama)
            for (tsv_tensor* t : {&L.wq, &L.wk}) {
                owned.emplace_back();
                if ((rc = unpermute_rotary_rows(p + (t == &L.wq ? "attn_q.weight" : "attn_k.weight"), *t, d.head_dim, owned.back())))
                    return rc;
                t->data = owned.back().data();
            }
    }
    d.layers = layers.data();
    // --kv-bits is a session option of the reference (crates/model-io/src/kv_quant.rs:48-72), not a property of
    // the file; here the process environment carries it: TSV_KV_BITS = off | 2 | 3 | 3.5 | 4
    if (const char* kvb = getenv("TSV_KV_BITS")) {
        const std::string v(kvb);
        if (v == "2") d.kv_k_bits = d.kv_v_bits = 2;
        else if (v == "3") d.kv_k_bits = d.kv_v_bits = 3;
        else if (v == "3.5") d.kv_k_bits = 3, d.kv_v_bits = 4;
        else if (v == "4") d.kv_k_bits = d.kv_v_bits = 4;
        else if (v != "off" && !v.empty()) {
            set_error("open_gguf: TSV_KV_BITS must be one of off|2|3|3.5|4");
            return TSV_ERR_INVALID;
        }
    }
    return tsv_open(&d, out);
}
