// Resident upload of one MoE layer's experts straight from MLX-format safetensors files.
//
// Replaces the SSD-streaming / LFU-cache pair of the reference (expert_stream.zig, expert_cache.zig, set up in
// model_registry.zig:255-329): instead of reading expert rows on demand, every (resident) expert of the layer is
// copied once from the memory-mapped file into HBM through dmoe_layer_create. File format (the reference's own
// test writes it, src/tests/numerical_equivalence_test.zig:29-88): 8-byte little-endian header length, a JSON
// object {name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}, then the tensor bytes;
// offsets are relative to the end of the header. Tensor names as in model_registry.zig:264-269:
//   model.layers.{i}.ffn.switch_mlp.{gate,up,down}_proj.{weight,scales,biases}
//   model.layers.{i}.ffn.shared_experts.{gate,up,down}_proj.{weight,scales,biases}   (optional)
// Host-only code; it lives in a .hip file so that the library keeps a single build rule.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "common.h"

namespace dmoe {

struct StTensor {
    std::string dtype;
    std::vector<long long> shape;
    const uint8_t *data = nullptr;
    size_t bytes = 0;
};

struct StFile {
    void *base = nullptr;
    size_t size = 0;
    ~StFile() {
        if (base) munmap(base, size);
    }
};

// ---- a JSON reader just large enough for the header -----------------------------------------------------
struct Json {
    const char *p, *end;
    bool ok = true;
    void ws() {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
    }
    bool eat(char c) {
        ws();
        if (p < end && *p == c) {
            ++p;
            return true;
        }
        return false;
    }
    std::string str() {
        ws();
        std::string s;
        if (p >= end || *p != '"') {
            ok = false;
            return s;
        }
        ++p;
        while (p < end && *p != '"') {
            if (*p == '\\' && p + 1 < end) { // escapes do not occur in tensor names; keep the escaped character
                ++p;
            }
            s.push_back(*p++);
        }
        if (p >= end) ok = false;
        else ++p;
        return s;
    }
    long long num() {
        ws();
        long long v = 0;
        bool any = false, neg = false;
        if (p < end && *p == '-') {
            neg = true;
            ++p;
        }
        while (p < end && *p >= '0' && *p <= '9') {
            v = v * 10 + (*p++ - '0');
            any = true;
        }
        if (!any) ok = false;
        return neg ? -v : v;
    }
    std::vector<long long> nums() {
        std::vector<long long> v;
        if (!eat('[')) {
            ok = false;
            return v;
        }
        if (eat(']')) return v;
        do v.push_back(num());
        while (ok && eat(','));
        if (!eat(']')) ok = false;
        return v;
    }
    void skip() { // any value
        ws();
        if (p >= end) {
            ok = false;
            return;
        }
        if (*p == '"') {
            str();
        } else if (*p == '{' || *p == '[') {
            const char close = *p == '{' ? '}' : ']';
            ++p;
            if (eat(close)) return;
            do {
                if (close == '}') {
                    str();
                    if (!eat(':')) ok = false;
                }
                skip();
            } while (ok && eat(','));
            if (!eat(close)) ok = false;
        } else {
            while (p < end && *p != ',' && *p != '}' && *p != ']') ++p;
        }
    }
};

static int index_file(const char *path, StFile *f, std::map<std::string, StTensor> *index) {
    int fd = open(path, O_RDONLY);
    DMOE_REQUIRE(fd >= 0, "safetensors: cannot open %s", path);
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size < 8) {
        close(fd);
        set_error("safetensors: %s is shorter than a header", path);
        return DMOE_ERR_INVALID;
    }
    f->size = (size_t)sb.st_size;
    f->base = mmap(nullptr, f->size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (f->base == MAP_FAILED) {
        f->base = nullptr;
        set_error("safetensors: mmap of %s failed", path);
        return DMOE_ERR_INVALID;
    }
    const uint8_t *b = (const uint8_t *)f->base;
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | b[i];
    DMOE_REQUIRE(hlen <= f->size - 8, "safetensors: header length %llu exceeds the file %s", (unsigned long long)hlen, path);
    const uint8_t *data = b + 8 + hlen;
    const size_t data_bytes = f->size - 8 - (size_t)hlen;
    Json j{(const char *)b + 8, (const char *)b + 8 + hlen};
    DMOE_REQUIRE(j.eat('{'), "safetensors: %s: header is not a JSON object", path);
    if (!j.eat('}')) {
        do {
            std::string name = j.str();
            if (!j.ok || !j.eat(':')) { j.ok = false; break; }
            if (name == "__metadata__") {
                j.skip();
                continue;
            }
            StTensor t;
            std::vector<long long> off;
            if (!j.eat('{')) { j.ok = false; break; }
            do {
                std::string key = j.str();
                if (!j.eat(':')) { j.ok = false; break; }
                if (key == "dtype") t.dtype = j.str();
                else if (key == "shape") t.shape = j.nums();
                else if (key == "data_offsets") off = j.nums();
                else j.skip();
            } while (j.ok && j.eat(','));
            if (!j.ok || !j.eat('}')) { j.ok = false; break; }
            if (off.size() != 2 || off[0] < 0 || off[1] < off[0] || (size_t)off[1] > data_bytes) {
                set_error("safetensors: %s: tensor %s has data_offsets outside the file", path, name.c_str());
                return DMOE_ERR_INVALID;
            }
            t.data = data + off[0];
            t.bytes = (size_t)(off[1] - off[0]);
            (*index)[name] = t;
        } while (j.ok && j.eat(','));
        DMOE_REQUIRE(j.ok && j.eat('}'), "safetensors: %s: malformed JSON header", path);
    }
    return DMOE_OK;
}

// a * b * c * d as a byte count; false if any factor is not positive or the product does not fit
static bool checked_bytes(long long a, long long b, long long c, long long d, size_t *out) {
    unsigned long long r = 1;
    for (long long f : {a, b, c, d}) {
        if (f <= 0 || __builtin_mul_overflow(r, (unsigned long long)f, &r)) return false;
    }
    if (r > (unsigned long long)SIZE_MAX / 2) return false;
    *out = (size_t)r;
    return true;
}

// one projection (weight + scales [+ biases]) of `prefix`, validated against the quantization parameters
static int find_proj(const std::map<std::string, StTensor> &index, const std::string &prefix, int mode, int bits,
                     int group, bool stacked, dmoe_qweight *q) {
    auto w = index.find(prefix + ".weight"), s = index.find(prefix + ".scales"), b = index.find(prefix + ".biases");
    DMOE_REQUIRE(w != index.end(), "safetensors: tensor %s.weight not found", prefix.c_str());
    const size_t nd = stacked ? 3 : 2;
    if (mode == DMOE_QUANT_NONE) { // unquantized experts: the bf16 matrix as it is
        const StTensor &tw = w->second;
        DMOE_REQUIRE(tw.shape.size() == nd, "safetensors: %s: expected a %zu-dimensional weight", prefix.c_str(), nd);
        DMOE_REQUIRE(tw.dtype == "BF16", "safetensors: %s.weight has dtype %s, expected BF16 (unquantized experts)",
                     prefix.c_str(), tw.dtype.c_str());
        const long long n = stacked ? tw.shape[0] : 1, rows = tw.shape[nd - 2], cols = tw.shape[nd - 1];
        size_t want_bytes = 0;
        DMOE_REQUIRE(n <= 1024 && rows <= INT32_MAX && cols <= INT32_MAX && checked_bytes(n, rows, cols, 2, &want_bytes) &&
                         tw.bytes == want_bytes,
                     "safetensors: %s.weight: bad shape or byte count", prefix.c_str());
        q->w = tw.data;
        q->scales = nullptr;
        q->biases = nullptr;
        q->n_mats = (int)n;
        q->rows = (int)rows;
        q->cols = (int)cols;
        q->mode = mode;
        q->bits = 16;
        q->group_size = 0;
        return DMOE_OK;
    }
    DMOE_REQUIRE(s != index.end(), "safetensors: tensor %s.scales not found (pass mode \"none\" for unquantized experts)",
                 prefix.c_str());
    // the quantization parameters come from the caller: check them before they divide anything
    DMOE_REQUIRE(bits == 4 || bits == 8, "safetensors: %s: bits must be 4 or 8, got %d", prefix.c_str(), bits);
    DMOE_REQUIRE(group == 32 || group == 64 || group == 128, "safetensors: %s: group size must be 32, 64 or 128, got %d",
                 prefix.c_str(), group);
    const StTensor &tw = w->second, &ts = s->second;
    DMOE_REQUIRE(tw.shape.size() == nd && ts.shape.size() == nd, "safetensors: %s: expected %zu-dimensional weight and scales",
                 prefix.c_str(), nd);
    DMOE_REQUIRE(tw.dtype == "U32", "safetensors: %s.weight has dtype %s, expected U32 (packed codes)", prefix.c_str(),
                 tw.dtype.c_str());
    const long long n = stacked ? tw.shape[0] : 1, rows = tw.shape[nd - 2], words = tw.shape[nd - 1];
    DMOE_REQUIRE(n >= 1 && n <= 1024 && rows >= 1 && rows <= INT32_MAX && words >= 1 && words <= INT32_MAX / 8,
                 "safetensors: %s: bad shape", prefix.c_str());
    const long long cols = words * 32 / bits;
    DMOE_REQUIRE(cols >= group && cols % group == 0, "safetensors: %s: bad shape", prefix.c_str());
    size_t w_bytes = 0, s_bytes = 0;
    DMOE_REQUIRE(checked_bytes(n, rows, words, 4, &w_bytes) && tw.bytes == w_bytes,
                 "safetensors: %s.weight: byte count does not match its shape", prefix.c_str());
    const char *want_s = mode == DMOE_QUANT_MXFP4 ? "U8" : "BF16";
    const size_t s_elem = mode == DMOE_QUANT_MXFP4 ? 1 : 2;
    DMOE_REQUIRE(ts.dtype == want_s, "safetensors: %s.scales has dtype %s, expected %s", prefix.c_str(), ts.dtype.c_str(), want_s);
    DMOE_REQUIRE((stacked ? ts.shape[0] : 1) == n && ts.shape[nd - 2] == rows && ts.shape[nd - 1] == cols / group &&
                     checked_bytes(n, rows, cols / group, (long long)s_elem, &s_bytes) && ts.bytes == s_bytes,
                 "safetensors: %s.scales does not match weight shape / group size %d", prefix.c_str(), group);
    q->w = tw.data;
    q->scales = ts.data;
    q->biases = nullptr;
    if (mode == DMOE_QUANT_AFFINE && b != index.end()) {
        const StTensor &tb = b->second;
        DMOE_REQUIRE(tb.dtype == "BF16" && tb.shape == ts.shape && tb.bytes == ts.bytes, "safetensors: %s.biases does not match scales",
                     prefix.c_str());
        q->biases = tb.data;
    }
    q->n_mats = (int)n;
    q->rows = (int)rows;
    q->cols = (int)cols;
    q->mode = mode;
    q->bits = bits;
    q->group_size = group;
    return DMOE_OK;
}

// keeps the experts whose mask byte is set, in increasing id order, in buffers of its own
struct Subset {
    std::vector<uint8_t> w, s, b;
    void take(dmoe_qweight *q, const uint8_t *mask, int n_total, int n_keep) {
        const bool plain = q->mode == DMOE_QUANT_NONE;
        const size_t wb = plain ? (size_t)q->rows * q->cols * 2 : (size_t)q->rows * (q->cols * q->bits / 32) * 4;
        const size_t sb = plain ? 0 : (size_t)q->rows * (q->cols / q->group_size) * (q->mode == DMOE_QUANT_MXFP4 ? 1 : 2);
        w.resize(wb * n_keep);
        s.resize(sb * n_keep);
        if (q->biases) b.resize(sb * n_keep);
        int slot = 0;
        for (int e = 0; e < n_total; ++e) {
            if (!mask[e]) continue;
            memcpy(w.data() + wb * slot, (const uint8_t *)q->w + wb * e, wb);
            if (sb) memcpy(s.data() + sb * slot, (const uint8_t *)q->scales + sb * e, sb);
            if (q->biases) memcpy(b.data() + sb * slot, (const uint8_t *)q->biases + sb * e, sb);
            ++slot;
        }
        q->w = w.data();
        if (sb) q->scales = s.data();
        if (q->biases) q->biases = b.data();
        q->n_mats = n_keep;
    }
};

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_layer_create_from_safetensors(dmoe_layer *out, const char *const *paths, int n_paths, int layer_idx,
                                                  const dmoe_safetensors_opts *o, dmoe_stream s) {
    DMOE_REQUIRE(out && paths && o, "layer_create_from_safetensors: null argument");
    out->ctx = nullptr;
    DMOE_REQUIRE(n_paths >= 1 && layer_idx >= 0, "layer_create_from_safetensors: need at least one file and a layer index >= 0");
    const int mode = dmoe_quant_mode_from_string(o->mode ? o->mode : "");
    DMOE_REQUIRE(mode == DMOE_QUANT_AFFINE || mode == DMOE_QUANT_MXFP4 || mode == DMOE_QUANT_NONE,
                 "layer_create_from_safetensors: mode must be \"affine\", \"mxfp4\" or \"none\"");
    std::vector<StFile> files((size_t)n_paths);
    std::map<std::string, StTensor> index;
    for (int i = 0; i < n_paths; ++i) {
        DMOE_REQUIRE(paths[i] != nullptr, "layer_create_from_safetensors: path %d is null", i);
        DMOE_TRY(index_file(paths[i], &files[i], &index));
    }
    const std::string base = "model.layers." + std::to_string(layer_idx) + ".ffn.";
    dmoe_layer_desc d;
    memset(&d, 0, sizeof(d));
    DMOE_TRY(find_proj(index, base + "switch_mlp.gate_proj", mode, o->bits, o->group_size, true, &d.gate));
    DMOE_TRY(find_proj(index, base + "switch_mlp.up_proj", mode, o->bits, o->group_size, true, &d.up));
    DMOE_TRY(find_proj(index, base + "switch_mlp.down_proj", mode, o->bits, o->group_size, true, &d.down));
    d.hidden = d.gate.cols;
    d.ffn = d.gate.rows;
    d.top_k = o->top_k;
    d.swiglu_limit = o->swiglu_limit;
    d.score_before_down = o->score_before_down;
    d.weight_source = DMOE_WEIGHTS_COPY_FROM_HOST;
    if (o->load_shared && index.count(base + "shared_experts.gate_proj.weight")) {
        // Without an explicit shared_mode the file decides, by the reference's rule (deepseek_v4_loader.zig:1890-1892):
        // biases present -> affine with the model's group size, scales only -> mxfp4 (group 32), neither -> float
        int smode;
        if (o->shared_mode) smode = dmoe_quant_mode_from_string(o->shared_mode);
        else if (!index.count(base + "shared_experts.gate_proj.scales")) smode = DMOE_QUANT_NONE;
        else smode = index.count(base + "shared_experts.gate_proj.biases") ? DMOE_QUANT_AFFINE : DMOE_QUANT_MXFP4;
        DMOE_REQUIRE(smode == DMOE_QUANT_AFFINE || smode == DMOE_QUANT_MXFP4 || smode == DMOE_QUANT_NONE,
                     "layer_create_from_safetensors: bad shared_mode");
        const int dbits = mode == DMOE_QUANT_NONE ? 4 : o->bits, dgroup = mode == DMOE_QUANT_NONE ? 64 : o->group_size;
        const int sbits = smode == DMOE_QUANT_NONE ? 16 : o->shared_bits ? o->shared_bits : dbits;
        const int sgroup = smode == DMOE_QUANT_MXFP4 ? 32 : o->shared_group_size ? o->shared_group_size : dgroup;
        DMOE_TRY(find_proj(index, base + "shared_experts.gate_proj", smode, sbits, sgroup, false, &d.shared_gate));
        DMOE_TRY(find_proj(index, base + "shared_experts.up_proj", smode, sbits, sgroup, false, &d.shared_up));
        DMOE_TRY(find_proj(index, base + "shared_experts.down_proj", smode, sbits, sgroup, false, &d.shared_down));
        d.has_shared = 1;
        d.shared_swiglu_limit = o->shared_swiglu_limit;
    }
    // Smelt: upload only the resident experts; router ids map to slots, unloaded ones to slot 0
    // (deepseek_v4_loader.zig:2151-2168)
    Subset sub[3];
    std::vector<int32_t> remap;
    DMOE_REQUIRE(d.up.n_mats == d.gate.n_mats && d.down.n_mats == d.gate.n_mats,
                 "layer_create_from_safetensors: gate / up / down hold %d / %d / %d experts", d.gate.n_mats, d.up.n_mats,
                 d.down.n_mats);
    if (o->resident_mask) {
        const int n_total = d.gate.n_mats;
        DMOE_REQUIRE(o->n_experts_total == n_total, "layer_create_from_safetensors: mask length %d, file holds %d experts",
                     o->n_experts_total, n_total);
        int n_keep = 0;
        for (int e = 0; e < n_total; ++e) n_keep += o->resident_mask[e] ? 1 : 0;
        DMOE_REQUIRE(n_keep >= 1, "layer_create_from_safetensors: the resident mask selects no expert");
        remap.resize((size_t)n_total);
        DMOE_TRY(dmoe_build_remap(remap.data(), o->resident_mask, n_total));
        dmoe_qweight *q[3] = {&d.gate, &d.up, &d.down};
        for (int i = 0; i < 3; ++i) sub[i].take(q[i], o->resident_mask, n_total, n_keep);
        d.remap = remap.data();
        d.n_experts_total = n_total;
    }
    return dmoe_layer_create(out, &d, s); // copies from the mapping; the files are unmapped on return
}
