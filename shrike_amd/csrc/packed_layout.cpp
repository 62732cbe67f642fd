// packed_experts/layout.json of a .gturbo model directory: a small JSON reader, the
// structural validator (sources/ShrikeFormat/GTurboPackedExpertsLayoutV1.swift:75-164), the
// manifest cross-check (:166-199) and the runtime view with the expert-offset look-up
// (sources/Shrike/Infrastructure/ModelIO/PackedExpertsLayout.swift:74-129,
// sources/Shrike/Runtime/Inference/ModelExpertIO.swift:69-94).
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstring>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

namespace {

// ---- JSON ---------------------------------------------------------------------------------

struct Json {
    enum Kind { Null, Bool, Integer, Real, String, Array, Object } kind = Null;
    bool boolean = false;
    bool negative = false;   // Integer: sign; magnitude in `magnitude`
    uint64_t magnitude = 0;
    std::string text;        // String
    std::vector<Json> items; // Array
    std::vector<std::pair<std::string, Json>> members;  // Object, in file order

    const Json *find(const char *key) const {
        const Json *hit = nullptr;
        for (const auto &m : members)
            if (m.first == key) hit = &m.second;  // the last of duplicate keys wins
        return hit;
    }
};

struct JsonReader {
    const char *p, *end, *begin;
    std::string error;
    int depth = 0;

    bool fail(const char *what) {
        if (error.empty()) error = std::string(what) + " at byte " + std::to_string(size_t(p - begin));
        return false;
    }
    JsonReader(const char *b, size_t n) : p(b), end(b + n), begin(b) {}

    void skip() {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
    }
    bool literal(const char *word) {
        const size_t n = strlen(word);
        if (size_t(end - p) < n || memcmp(p, word, n) != 0) return fail("unexpected token");
        p += n;
        return true;
    }
    static void append_utf8(std::string &out, uint32_t cp) {
        if (cp < 0x80) out += char(cp);
        else if (cp < 0x800) { out += char(0xC0 | (cp >> 6)); out += char(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) { out += char(0xE0 | (cp >> 12)); out += char(0x80 | ((cp >> 6) & 0x3F)); out += char(0x80 | (cp & 0x3F)); }
        else { out += char(0xF0 | (cp >> 18)); out += char(0x80 | ((cp >> 12) & 0x3F)); out += char(0x80 | ((cp >> 6) & 0x3F)); out += char(0x80 | (cp & 0x3F)); }
    }
    bool hex4(uint32_t &out) {
        if (end - p < 4) return fail("short \\u escape");
        out = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = *p++;
            out <<= 4;
            if (c >= '0' && c <= '9') out |= uint32_t(c - '0');
            else if (c >= 'a' && c <= 'f') out |= uint32_t(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') out |= uint32_t(c - 'A' + 10);
            else return fail("bad \\u escape");
        }
        return true;
    }
    bool string(std::string &out) {
        if (p >= end || *p != '"') return fail("expected a string");
        ++p;
        while (p < end && *p != '"') {
            const unsigned char c = static_cast<unsigned char>(*p++);
            if (c < 0x20) return fail("control character in a string");
            if (c != '\\') { out += char(c); continue; }
            if (p >= end) return fail("short escape");
            const char e = *p++;
            switch (e) {
                case '"': out += '"'; break;
                case '\\': out += '\\'; break;
                case '/': out += '/'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'n': out += '\n'; break;
                case 'r': out += '\r'; break;
                case 't': out += '\t'; break;
                case 'u': {
                    uint32_t cp;
                    if (!hex4(cp)) return false;
                    if (cp >= 0xD800 && cp < 0xDC00) {  // a surrogate pair
                        uint32_t lo;
                        if (end - p < 2 || p[0] != '\\' || p[1] != 'u') return fail("lone surrogate");
                        p += 2;
                        if (!hex4(lo)) return false;
                        if (lo < 0xDC00 || lo > 0xDFFF) return fail("lone surrogate");
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
                        return fail("lone surrogate");
                    }
                    append_utf8(out, cp);
                    break;
                }
                default: return fail("bad escape");
            }
        }
        if (p >= end) return fail("unterminated string");
        ++p;
        return true;
    }
    bool number(Json &out) {
        const char *start = p;
        bool neg = false;
        if (p < end && *p == '-') { neg = true; ++p; }
        if (p >= end || !isdigit(static_cast<unsigned char>(*p))) return fail("bad number");
        if (*p == '0' && p + 1 < end && isdigit(static_cast<unsigned char>(p[1]))) return fail("leading zero");
        uint64_t mag = 0;
        bool overflow = false;
        while (p < end && isdigit(static_cast<unsigned char>(*p))) {
            const uint64_t d = uint64_t(*p - '0');
            if (mag > (UINT64_MAX - d) / 10) overflow = true;
            mag = mag * 10 + d;
            ++p;
        }
        bool real = false;
        if (p < end && *p == '.') {
            real = true;
            ++p;
            if (p >= end || !isdigit(static_cast<unsigned char>(*p))) return fail("bad fraction");
            while (p < end && isdigit(static_cast<unsigned char>(*p))) ++p;
        }
        if (p < end && (*p == 'e' || *p == 'E')) {
            real = true;
            ++p;
            if (p < end && (*p == '+' || *p == '-')) ++p;
            if (p >= end || !isdigit(static_cast<unsigned char>(*p))) return fail("bad exponent");
            while (p < end && isdigit(static_cast<unsigned char>(*p))) ++p;
        }
        out.kind = (real || overflow) ? Json::Real : Json::Integer;
        out.negative = neg && mag != 0;
        out.magnitude = mag;
        out.text.assign(start, size_t(p - start));
        return true;
    }
    bool value(Json &out) {
        if (++depth > 64) return fail("nesting too deep");
        skip();
        if (p >= end) return fail("unexpected end");
        bool ok = true;
        switch (*p) {
            case '{': {
                out.kind = Json::Object;
                ++p;
                skip();
                if (p < end && *p == '}') { ++p; break; }
                for (;;) {
                    skip();
                    std::string key;
                    if (!string(key)) return false;
                    skip();
                    if (p >= end || *p != ':') return fail("expected ':'");
                    ++p;
                    Json v;
                    if (!value(v)) return false;
                    out.members.emplace_back(std::move(key), std::move(v));
                    skip();
                    if (p < end && *p == ',') { ++p; continue; }
                    if (p < end && *p == '}') { ++p; break; }
                    return fail("expected ',' or '}'");
                }
                break;
            }
            case '[': {
                out.kind = Json::Array;
                ++p;
                skip();
                if (p < end && *p == ']') { ++p; break; }
                for (;;) {
                    Json v;
                    if (!value(v)) return false;
                    out.items.push_back(std::move(v));
                    skip();
                    if (p < end && *p == ',') { ++p; continue; }
                    if (p < end && *p == ']') { ++p; break; }
                    return fail("expected ',' or ']'");
                }
                break;
            }
            case '"': out.kind = Json::String; ok = string(out.text); break;
            case 't': out.kind = Json::Bool; out.boolean = true; ok = literal("true"); break;
            case 'f': out.kind = Json::Bool; out.boolean = false; ok = literal("false"); break;
            case 'n': out.kind = Json::Null; ok = literal("null"); break;
            default: ok = number(out); break;
        }
        --depth;
        return ok;
    }
    bool document(Json &out) {
        if (!value(out)) return false;
        skip();
        if (p != end) return fail("trailing bytes");
        return true;
    }
};

// ---- the layout -----------------------------------------------------------------------------

struct Tensor {
    uint64_t offset = 0, size = 0;
    std::string dtype;
    std::vector<uint32_t> shape;
    bool has_bits = false;
    int64_t bits = 0;
};

struct Expert {
    bool has_expert = false, has_rank = false;
    int64_t expert = 0, physical_rank = 0;  // as written; resolved below
    uint64_t offset = 0, size = 0;
    std::map<std::string, Tensor> tensors;
    int64_t logical = 0, physical = 0;
};

struct Layer {
    int64_t layer = 0;
    std::string file;
    std::vector<Expert> experts;
};

}  // namespace

struct shrike_packed_layout {
    uint64_t expert_stride = 0;
    int64_t num_layers = 0, experts_per_layer = 0;
    std::vector<Layer> layers;
};

namespace {

// Decoding the wire form: a missing or mistyped required key is a decoding error
// (GTurboPackedExpertsLayoutV1.swift:65-72).
struct DecodeError {
    std::string path, reason;
};

bool as_u64(const Json *j, uint64_t &out) {
    if (!j || j->kind != Json::Integer || j->negative) return false;
    out = j->magnitude;
    return true;
}
bool as_i64(const Json *j, int64_t &out) {
    if (!j || j->kind != Json::Integer) return false;
    if (j->negative) {
        if (j->magnitude > uint64_t(INT64_MAX) + 1u) return false;
        out = j->magnitude == uint64_t(INT64_MAX) + 1u ? INT64_MIN : -int64_t(j->magnitude);
    } else {
        if (j->magnitude > uint64_t(INT64_MAX)) return false;
        out = int64_t(j->magnitude);
    }
    return true;
}

#define NEED(cond, where, why)            \
    do {                                  \
        if (!(cond)) {                    \
            err.path = (where);           \
            err.reason = (why);           \
            return false;                 \
        }                                 \
    } while (0)

bool decode_tensor(const Json &j, const std::string &at, Tensor &t, DecodeError &err) {
    NEED(j.kind == Json::Object, at, "expected an object");
    NEED(as_u64(j.find("offset"), t.offset), at + ".offset", "expected an unsigned integer");
    NEED(as_u64(j.find("size"), t.size), at + ".size", "expected an unsigned integer");
    const Json *dtype = j.find("dtype");
    NEED(dtype && dtype->kind == Json::String, at + ".dtype", "expected a string");
    t.dtype = dtype->text;
    const Json *shape = j.find("shape");
    NEED(shape && shape->kind == Json::Array, at + ".shape", "expected an array");
    for (const Json &d : shape->items) {
        uint64_t v;
        NEED(as_u64(&d, v) && v <= UINT32_MAX, at + ".shape", "expected 32-bit unsigned integers");
        t.shape.push_back(uint32_t(v));
    }
    const Json *bits = j.find("bits");
    if (bits && bits->kind != Json::Null) {
        NEED(as_i64(bits, t.bits), at + ".bits", "expected an integer");
        t.has_bits = true;
    }
    return true;
}

bool decode_expert(const Json &j, const std::string &at, Expert &e, DecodeError &err) {
    NEED(j.kind == Json::Object, at, "expected an object");
    const Json *id = j.find("expert");
    if (id && id->kind != Json::Null) {
        NEED(as_i64(id, e.expert), at + ".expert", "expected an integer");
        e.has_expert = true;
    }
    const Json *rank = j.find("physicalRank");
    if (rank && rank->kind != Json::Null) {
        NEED(as_i64(rank, e.physical_rank), at + ".physicalRank", "expected an integer");
        e.has_rank = true;
    }
    NEED(as_u64(j.find("offset"), e.offset), at + ".offset", "expected an unsigned integer");
    NEED(as_u64(j.find("size"), e.size), at + ".size", "expected an unsigned integer");
    const Json *tensors = j.find("tensors");
    NEED(tensors && tensors->kind == Json::Object, at + ".tensors", "expected an object");
    for (const auto &m : tensors->members) {
        Tensor t;
        if (!decode_tensor(m.second, at + ".tensors." + m.first, t, err)) return false;
        e.tensors[m.first] = std::move(t);
    }
    return true;
}

bool decode_wire(const Json &root, shrike_packed_layout &out, DecodeError &err) {
    NEED(root.kind == Json::Object, "layout", "expected an object");
    NEED(as_u64(root.find("expertStride"), out.expert_stride), "expertStride", "expected an unsigned integer");
    NEED(as_i64(root.find("numLayers"), out.num_layers), "numLayers", "expected an integer");
    NEED(as_i64(root.find("expertsPerLayer"), out.experts_per_layer), "expertsPerLayer", "expected an integer");
    const Json *layers = root.find("layers");
    NEED(layers && layers->kind == Json::Array, "layers", "expected an array");
    for (size_t i = 0; i < layers->items.size(); ++i) {
        const Json &j = layers->items[i];
        const std::string at = "layers[" + std::to_string(i) + "]";
        NEED(j.kind == Json::Object, at, "expected an object");
        Layer layer;
        NEED(as_i64(j.find("layer"), layer.layer), at + ".layer", "expected an integer");
        const Json *file = j.find("file");
        NEED(file && file->kind == Json::String, at + ".file", "expected a string");
        layer.file = file->text;
        const Json *experts = j.find("experts");
        NEED(experts && experts->kind == Json::Array, at + ".experts", "expected an array");
        for (size_t k = 0; k < experts->items.size(); ++k) {
            Expert e;
            if (!decode_expert(experts->items[k], at + ".experts[" + std::to_string(k) + "]", e, err)) return false;
            layer.experts.push_back(std::move(e));
        }
        out.layers.push_back(std::move(layer));
    }
    return true;
}
#undef NEED

int invalid(const std::string &field, const std::string &reason) {
    set_error("layout.json: invalid %s: %s", field.c_str(), reason.c_str());
    return EINVAL;
}

// GTurboPathValidator.validateBasename (sources/ShrikeFormat/GTurboFormatV1.swift:58-77)
const char *basename_fault(const std::string &name) {
    if (name.empty() || name[0] == '/' || name.find('\0') != std::string::npos) return "unsafe relative path";
    size_t start = 0;
    for (;;) {
        const size_t slash = name.find('/', start);
        const std::string part = name.substr(start, slash == std::string::npos ? std::string::npos : slash - start);
        if (part.empty() || part == "." || part == "..") return "non-canonical path";
        if (slash == std::string::npos) break;
        start = slash + 1;
    }
    if (name.find('/') != std::string::npos) return "expected basename";
    return nullptr;
}

// appleFilesystemKey (GTurboFormatV1.swift:53-56) lower-cases the canonically composed name.
// Here: ASCII letters are folded; bytes outside ASCII are compared as they are written.
std::string filesystem_key(const std::string &name) {
    std::string key = name;
    for (char &c : key)
        if (c >= 'A' && c <= 'Z') c = char(c - 'A' + 'a');
    return key;
}

// GTurboV1StructuralValidator.validate, in the reference's order of checks.
int validate(shrike_packed_layout &layout) {
    if (!(layout.num_layers > 0 && layout.experts_per_layer > 0 && layout.expert_stride > 0
          && layout.expert_stride % SHRIKE_LAYOUT_ALIGNMENT_BYTES == 0
          && int64_t(layout.layers.size()) == layout.num_layers))
        return invalid("layout", "invalid dimensions or stride");
    std::set<int64_t> layer_ids;
    std::set<std::string> layer_files;
    for (Layer &layer : layout.layers) {
        if (!(layer.layer >= 0 && layer.layer < layout.num_layers && layer_ids.insert(layer.layer).second))
            return invalid("layout.layers", "duplicate or invalid layer");
        const std::string file_field = "layout.layers[" + std::to_string(layer.layer) + "].file";
        if (const char *fault = basename_fault(layer.file)) return invalid(file_field, fault);
        const std::string key = filesystem_key(layer.file);
        if (key == "layout.json") return invalid(file_field, "reserved packed-expert filename");
        if (!layer_files.insert(key).second) return invalid(file_field, "duplicate layer filename");
        const std::string experts_field = "layout.layers[" + std::to_string(layer.layer) + "].experts";
        // a dense-MLP layer carries an empty expert list (and no layer file)
        if (!(int64_t(layer.experts.size()) == layout.experts_per_layer || layer.experts.empty()))
            return invalid(experts_field, "wrong expert count");
        size_t explicit_ids = 0;
        for (const Expert &e : layer.experts) explicit_ids += e.has_expert ? 1 : 0;
        if (explicit_ids != 0 && explicit_ids != layer.experts.size())
            return invalid(experts_field, "expert ids must be either all explicit or all positional");
        std::set<int64_t> logical_ids, physical_ranks;
        std::set<uint64_t> offsets;
        for (size_t position = 0; position < layer.experts.size(); ++position) {
            Expert &e = layer.experts[position];
            e.logical = e.has_expert ? e.expert : int64_t(position);
            e.physical = e.has_rank ? e.physical_rank : e.logical;
            if (!(e.logical >= 0 && e.logical < layout.experts_per_layer && e.physical >= 0
                  && e.physical < layout.experts_per_layer && logical_ids.insert(e.logical).second
                  && physical_ranks.insert(e.physical).second && offsets.insert(e.offset).second))
                return invalid(experts_field, "duplicate or invalid expert mapping");
            unsigned __int128 expected = (unsigned __int128)uint64_t(e.physical) * layout.expert_stride;
            if (expected > UINT64_MAX) {
                set_error("layout.json: arithmetic overflow in expert.offset");
                return EINVAL;
            }
            const std::string expert_field = "expert[" + std::to_string(e.logical) + "]";
            if (!(e.offset == uint64_t(expected) && e.size == layout.expert_stride))
                return invalid(expert_field, "offset or size does not match physical rank");
            struct Range { uint64_t start, end; const std::string *name; };
            std::vector<Range> ranges;
            for (const auto &named : e.tensors) {
                const Tensor &t = named.second;
                const std::string tensor_field = expert_field + ".tensors." + named.first;
                bool shape_ok = !t.shape.empty();
                for (uint32_t d : t.shape) shape_ok = shape_ok && d > 0;
                if (!((t.dtype == "U32" || t.dtype == "BF16") && !named.first.empty() && t.size > 0 && shape_ok
                      && (!t.has_bits || (t.bits > 0 && t.bits <= 32))))
                    return invalid(tensor_field, "invalid dtype or shape");
                if (t.offset > UINT64_MAX - t.size) {
                    set_error("layout.json: arithmetic overflow in tensor.%s.range", named.first.c_str());
                    return EINVAL;
                }
                if (t.offset + t.size > e.size) return invalid(tensor_field, "range exceeds expert blob");
                ranges.push_back({t.offset, t.offset + t.size, &named.first});
            }
            std::sort(ranges.begin(), ranges.end(), [](const Range &a, const Range &b) {
                return a.start == b.start ? a.end < b.end : a.start < b.start;
            });
            for (size_t i = 0; i + 1 < ranges.size(); ++i)
                if (ranges[i].end > ranges[i + 1].start)
                    return invalid(expert_field + ".tensors",
                                   "overlapping ranges " + *ranges[i].name + " and " + *ranges[i + 1].name);
        }
    }
    // the runtime view (PackedExpertsLayout.swift:104-121): layers by id, experts by logical id
    std::sort(layout.layers.begin(), layout.layers.end(), [](const Layer &a, const Layer &b) { return a.layer < b.layer; });
    for (Layer &layer : layout.layers)
        std::sort(layer.experts.begin(), layer.experts.end(), [](const Expert &a, const Expert &b) { return a.logical < b.logical; });
    return 0;
}

const Expert *expert_at(const shrike_packed_layout *layout, int layer, int expert) {
    if (!layout) {
        set_error("layout is NULL");
        return nullptr;
    }
    if (layer < 0 || size_t(layer) >= layout->layers.size()) {
        set_error("expert layout has %zu layers; layer %d is out of range", layout->layers.size(), layer);
        return nullptr;
    }
    const Layer &l = layout->layers[size_t(layer)];
    if (expert < 0 || size_t(expert) >= l.experts.size()) {
        set_error("layer %d has %zu experts; expert %d is out of range", layer, l.experts.size(), expert);
        return nullptr;
    }
    return &l.experts[size_t(expert)];
}

}  // namespace

extern "C" {

shrike_packed_layout *shrike_packed_layout_decode(const char *json, size_t bytes, int *out_errno) {
    auto fail = [&](int err) -> shrike_packed_layout * {
        if (out_errno) *out_errno = err;
        return nullptr;
    };
    if (out_errno) *out_errno = 0;
    if (!json) {
        set_error("layout.json: no data");
        return fail(EINVAL);
    }
    JsonReader reader(json, bytes);
    Json root;
    if (!reader.document(root)) {
        set_error("layout.json: invalid packed_experts/layout.json: %s", reader.error.c_str());
        return fail(EINVAL);
    }
    std::unique_ptr<shrike_packed_layout> layout(new shrike_packed_layout());
    DecodeError err;
    if (!decode_wire(root, *layout, err)) {
        set_error("layout.json: invalid packed_experts/layout.json: %s: %s", err.path.c_str(), err.reason.c_str());
        return fail(EINVAL);
    }
    if (int rc = validate(*layout)) return fail(rc);
    return layout.release();
}

shrike_packed_layout *shrike_packed_layout_load(const char *model_dir, uint64_t max_bytes, int *out_errno) {
    auto fail = [&](int err) -> shrike_packed_layout * {
        if (out_errno) *out_errno = err;
        return nullptr;
    };
    if (out_errno) *out_errno = 0;
    if (!model_dir) {
        set_error("model directory is NULL");
        return fail(EINVAL);
    }
    if (max_bytes == 0) max_bytes = SHRIKE_LAYOUT_MAX_BYTES;
    const std::string relative = "packed_experts/layout.json";
    const std::string path = std::string(model_dir) + "/" + relative;
    const int fd = open(path.c_str(), O_RDONLY | O_NONBLOCK | O_NOFOLLOW | O_CLOEXEC);  // GTurboModelDirectory.swift:47-48
    if (fd < 0) {
        const int err = errno;
        set_error("missing file %s: %s", relative.c_str(), strerror(err));
        return fail(err);
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || !S_ISREG(st.st_mode)) {
        const int err = errno ? errno : EINVAL;
        close(fd);
        set_error("fstat(%s) failed or it is not a regular file", relative.c_str());
        return fail(err);
    }
    if (uint64_t(st.st_size) > max_bytes) {
        close(fd);
        set_error("%s size %llu exceeds metadata cap %llu", relative.c_str(), (unsigned long long)st.st_size,
                  (unsigned long long)max_bytes);
        return fail(EFBIG);
    }
    std::string data(size_t(st.st_size), '\0');
    size_t total = 0;
    while (total < data.size()) {
        const ssize_t got = pread(fd, &data[total], data.size() - total, off_t(total));
        if (got < 0 && errno == EINTR) continue;
        if (got <= 0) {
            const int err = got < 0 ? errno : EIO;
            close(fd);
            set_error("pread(%s) failed: %s", relative.c_str(), strerror(err));
            return fail(err);
        }
        total += size_t(got);
    }
    close(fd);
    return shrike_packed_layout_decode(data.data(), data.size(), out_errno);
}

void shrike_packed_layout_destroy(shrike_packed_layout *layout) { delete layout; }

uint64_t shrike_packed_layout_expert_stride(const shrike_packed_layout *layout) { return layout ? layout->expert_stride : 0; }
int shrike_packed_layout_num_layers(const shrike_packed_layout *layout) { return layout ? int(layout->num_layers) : 0; }
int shrike_packed_layout_experts_per_layer(const shrike_packed_layout *layout) {
    return layout ? int(layout->experts_per_layer) : 0;
}

int shrike_packed_layout_layer(const shrike_packed_layout *layout, int index, int *layer_id, const char **file,
                               int *expert_count) {
    SHRIKE_REQUIRE(layout != nullptr, "layout is NULL");
    SHRIKE_REQUIRE(index >= 0 && size_t(index) < layout->layers.size(), "expert layout has %zu layers; layer %d is out of range",
                   layout->layers.size(), index);
    const Layer &l = layout->layers[size_t(index)];
    if (layer_id) *layer_id = int(l.layer);
    if (file) *file = l.file.c_str();
    if (expert_count) *expert_count = int(l.experts.size());
    return 0;
}

int shrike_packed_layout_expert(const shrike_packed_layout *layout, int layer, int expert, shrike_packed_expert *out) {
    const Expert *e = expert_at(layout, layer, expert);
    if (!e) return layout ? ERANGE : EINVAL;
    SHRIKE_REQUIRE(out != nullptr, "out is NULL");
    out->expert = int32_t(e->logical);
    out->physical_rank = int32_t(e->physical);
    out->offset = e->offset;
    out->size = e->size;
    out->tensor_count = uint32_t(e->tensors.size());
    return 0;
}

int shrike_packed_layout_tensor(const shrike_packed_layout *layout, int layer, int expert, const char *role,
                                shrike_packed_tensor *out) {
    const Expert *e = expert_at(layout, layer, expert);
    if (!e) return layout ? ERANGE : EINVAL;
    SHRIKE_REQUIRE(role != nullptr && out != nullptr, "role or out is NULL");
    const auto it = e->tensors.find(role);
    if (it == e->tensors.end()) {
        set_error("expert %d of layer %d has no tensor %s", expert, layer, role);
        return ENOENT;
    }
    const Tensor &t = it->second;
    memset(out, 0, sizeof *out);
    out->offset = t.offset;
    out->size = t.size;
    strncpy(out->dtype, t.dtype.c_str(), sizeof out->dtype - 1);
    out->rank = uint32_t(t.shape.size());
    for (size_t i = 0; i < t.shape.size() && i < 4; ++i) out->shape[i] = t.shape[i];
    out->bits = t.has_bits ? int32_t(t.bits) : 0;
    return 0;
}

int shrike_packed_layout_expert_offsets(const shrike_packed_layout *layout, int layer, int experts_have_additive_biases,
                                        shrike_expert_offsets *out) {
    const Expert *e = expert_at(layout, layer, 0);
    if (!e) return layout ? ERANGE : EINVAL;
    SHRIKE_REQUIRE(out != nullptr, "out is NULL");
    auto offset = [&](const char *role) -> uint32_t {
        const auto it = e->tensors.find(role);
        return it == e->tensors.end() ? 0u : uint32_t(it->second.offset);
    };
    if (experts_have_additive_biases) {
        for (const char *role : {"gate_bias", "up_bias", "down_bias"})
            SHRIKE_REQUIRE(e->tensors.count(role) != 0, "layer %d expert blob is missing %s", layer, role);
    }
    out->gate_w_off = offset("gate"); out->gate_s_off = offset("gate_scales"); out->gate_b_off = offset("gate_biases");
    out->up_w_off = offset("up"); out->up_s_off = offset("up_scales"); out->up_b_off = offset("up_biases");
    out->down_w_off = offset("down"); out->down_s_off = offset("down_scales"); out->down_b_off = offset("down_biases");
    out->gate_ab_off = offset("gate_bias"); out->up_ab_off = offset("up_bias"); out->down_ab_off = offset("down_bias");
    return 0;
}

int shrike_packed_layout_cross_validate(const shrike_packed_layout *layout, int manifest_num_layers,
                                        int manifest_experts_per_layer, uint64_t manifest_expert_stride,
                                        const char *const *manifest_paths, const uint64_t *manifest_sizes,
                                        size_t manifest_file_count) {
    SHRIKE_REQUIRE(layout != nullptr, "layout is NULL");
    SHRIKE_REQUIRE(manifest_file_count == 0 || (manifest_paths && manifest_sizes), "manifest file list is NULL");
    if (!(manifest_num_layers == layout->num_layers && manifest_experts_per_layer == layout->experts_per_layer
          && manifest_expert_stride == layout->expert_stride))
        return invalid("manifest/layout", "dimension mismatch");
    const unsigned __int128 layer_size = (unsigned __int128)uint64_t(layout->experts_per_layer) * layout->expert_stride;
    if (layer_size > UINT64_MAX) {
        set_error("layout.json: arithmetic overflow in layout.layerSize");
        return EINVAL;
    }
    for (const Layer &l : layout->layers) {
        if (l.experts.empty()) continue;
        const std::string path = "packed_experts/" + l.file;
        bool found = false;
        for (size_t i = 0; i < manifest_file_count && !found; ++i)
            found = path == manifest_paths[i] && manifest_sizes[i] == uint64_t(layer_size);
        if (!found) return invalid("manifest.files." + path, "missing or wrong layer size");
    }
    return 0;
}

}  // extern "C"
