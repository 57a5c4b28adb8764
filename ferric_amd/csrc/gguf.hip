// GGUF container reader (host code): header, metadata, tensor table, and zero-copy access to a tensor's raw
// bytes in the mapped file, so that a quantized weight goes file -> HBM with no intermediate copy or repack.
//
// Follows crates/ferric-gguf/src/lib.rs: the bounds-safe cursor (:56-104, every read past the end marks the
// parse failed instead of faulting), `parse` (:105-132), `check_declared_strides` (:387-431), `type_size`
// (:460-484) and `Gguf::raw` / `GgufFile::raw` (:443-449, :566-573). Not restated: `resolve_ambiguous_types`
// (:330-385), which settles the contested type ids 41 / 42 of formats this library has no kernels for; such
// tensors are listed with the id the file declares and cannot be made into weights here.
#include "common.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace {

enum Kind : int { K_U = 0, K_I = 1, K_F = 2, K_BOOL = 3, K_STR = 4, K_ARR = 5 };

struct Meta {
    int kind = K_U;
    uint64_t u = 0;      // U, Bool
    int64_t i = 0;       // I
    double f = 0;        // F
    std::string s;       // Str
    std::vector<Meta> a; // Arr
};

struct TensorInfo {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t ggml_type = 0;
    uint64_t offset = 0;
};

// A window [at, end) over the mapped file that only moves forward. Every read is checked against what is left; the first
// read that does not fit sets `bad` and from then on every read yields zeros, so a parser can run to its end and ask once.
// (Bounds behaviour of crates/ferric-gguf/src/lib.rs:56-104: a short or hostile header is refused, never read past.)
struct Window {
    const uint8_t* at;
    const uint8_t* end;
    bool bad = false;
    size_t left() const { return (size_t)(end - at); }
    const uint8_t* bytes(uint64_t k) {
        if (bad || k > left()) { bad = true; return nullptr; }
        const uint8_t* s = at;
        at += (size_t)k;
        return s;
    }
    template <class T> T scalar() {
        T v{};
        if (const uint8_t* s = bytes(sizeof(T))) memcpy(&v, s, sizeof(T));
        return v;
    }
    // u64 length + bytes. The length is compared with what is left BEFORE anything is sized by it: a length field of
    // 2^60 in a 1 KiB file is an error, not an allocation.
    std::string text() {
        const uint64_t len = scalar<uint64_t>();
        const uint8_t* s = bytes(len);
        return s ? std::string((const char*)s, (size_t)len) : std::string();
    }
};

// One metadata value of GGUF value type `ty` (0..12; 9 = array of one element type, nested at most 8 deep).
Meta read_value(Window& w, uint32_t ty, int depth = 0) {
    Meta m;
    auto as_u = [&](uint64_t v) { m.kind = K_U; m.u = v; };
    auto as_i = [&](int64_t v) { m.kind = K_I; m.i = v; };
    auto as_f = [&](double v) { m.kind = K_F; m.f = v; };
    switch (ty) {
        case 0: as_u(w.scalar<uint8_t>()); break;
        case 1: as_i(w.scalar<int8_t>()); break;
        case 2: as_u(w.scalar<uint16_t>()); break;
        case 3: as_i(w.scalar<int16_t>()); break;
        case 4: as_u(w.scalar<uint32_t>()); break;
        case 5: as_i(w.scalar<int32_t>()); break;
        case 6: as_f(w.scalar<float>()); break;
        case 7: m.kind = K_BOOL; m.u = w.scalar<uint8_t>() != 0; break;
        case 8: m.kind = K_STR; m.s = w.text(); break;
        case 9: {
            m.kind = K_ARR;
            const uint32_t elem = w.scalar<uint32_t>();
            const uint64_t count = w.scalar<uint64_t>();
            // no element type is shorter than a byte, so more elements than bytes left cannot be a real array
            if (count > w.left() || depth > 8) { w.bad = true; break; }
            m.a.reserve((size_t)count);
            for (uint64_t k = 0; k < count && !w.bad; k++) m.a.push_back(read_value(w, elem, depth + 1));
            break;
        }
        case 10: as_u(w.scalar<uint64_t>()); break;
        case 11: as_i(w.scalar<int64_t>()); break;
        case 12: as_f(w.scalar<double>()); break;
        default: w.bad = true; break;
    }
    return m;
}

// On-disk size of n elements of ggml type ty, the reference's whole table (lib.rs:460-484): the stride check
// needs the size of every tensor in the file, not only of the formats this library computes with.
bool type_size_all(uint32_t ty, uint64_t n, uint64_t* out) {
    switch (ty) {
        case 0: *out = n * 4; return true;            // F32
        case 1: *out = n * 2; return true;            // F16
        case 30: *out = n * 2; return true;           // BF16
        case 8: *out = n / 32 * 34; return true;      // Q8_0
        case 2: *out = n / 32 * 18; return true;      // Q4_0
        case 3: *out = n / 32 * 20; return true;      // Q4_1
        case 6: *out = n / 32 * 22; return true;      // Q5_0
        case 7: *out = n / 32 * 24; return true;      // Q5_1
        case 12: *out = n / 256 * 144; return true;   // Q4_K
        case 13: *out = n / 256 * 176; return true;   // Q5_K
        case 14: *out = n / 256 * 210; return true;   // Q6_K
        case 20: *out = n / 32 * 18; return true;     // IQ4_NL
        case 23: *out = n / 256 * 136; return true;   // IQ4_XS
        case 35: *out = n / 256 * 66; return true;    // TQ2_0
        case 39: *out = n / 32 * 17; return true;     // MXFP4
        case 41: *out = n / 128 * 18; return true;    // Q1_0
        case 42: *out = n / 128 * 34; return true;    // Q2_0 (PrismML layout)
        case 1042: *out = n / 128 * 129; return true; // F8_E4M3_B128 (internal id)
        default: return false;
    }
}

uint64_t numel(const TensorInfo& t) {
    uint64_t n = 1;
    for (uint64_t d : t.dims) n *= d;
    return n;
}

// lib.rs:387-431. Returns "" or the refusal text.
std::string check_declared_strides(const std::vector<TensorInfo>& tensors, uint64_t data_len, uint64_t align) {
    std::vector<const TensorInfo*> by(tensors.size());
    for (size_t i = 0; i < tensors.size(); i++) by[i] = &tensors[i];
    std::stable_sort(by.begin(), by.end(), [](const TensorInfo* a, const TensorInfo* b) { return a->offset < b->offset; });
    // a header probe holds a prefix of the file: if the buffer ends before the last tensor begins, the last
    // tensor's bound is unknowable and is the one check that is skipped
    const bool have_full_data = by.empty() || data_len >= by.back()->offset;
    char buf[1024];
    for (size_t i = 0; i < by.size(); i++) {
        const TensorInfo& t = *by[i];
        const uint64_t n = numel(t);
        uint64_t sz;
        if (!type_size_all(t.ggml_type, n, &sz)) continue;   // an unknown type is a separate, already loud failure
        uint64_t limit;
        if (i + 1 < by.size()) limit = by[i + 1]->offset;
        else if (have_full_data) limit = data_len;
        else continue;
        const uint64_t avail = limit > t.offset ? limit - t.offset : 0;
        if (sz > avail) {
            snprintf(buf, sizeof buf,
                     "tensor '%s' (ggml type %u, %llu elements) needs %llu bytes by this reader's block layout, but the file "
                     "leaves only %llu before the next tensor. The type id's layout here disagrees with the writer's, so "
                     "reading it would silently return garbage at the wrong stride rather than fail. Refusing to load.",
                     t.name.c_str(), t.ggml_type, (unsigned long long)n, (unsigned long long)sz, (unsigned long long)avail);
            return buf;
        }
        // padding between tensors is legal; a gap far beyond alignment means the stride is too small
        const uint64_t slack = std::max<uint64_t>(align, 64) * 4;
        if (i + 1 < by.size() && avail > sz + slack && avail > sz * 2) {
            snprintf(buf, sizeof buf,
                     "tensor '%s' (ggml type %u, %llu elements) is %llu bytes by this reader's block layout, but the file "
                     "reserves %llu for it - more than twice as much, and far beyond alignment padding. This reader's "
                     "stride for that type id is too small, which reads a short prefix of every block. Refusing to load.",
                     t.name.c_str(), t.ggml_type, (unsigned long long)n, (unsigned long long)sz, (unsigned long long)avail);
            return buf;
        }
    }
    return {};
}

}  // namespace

struct fhip_gguf {
    const uint8_t* bytes = nullptr;
    size_t len = 0;
    void* map = nullptr;        // non-null: the file mapping this handle owns
    size_t map_len = 0;
    uint32_t version = 0;
    std::vector<std::pair<std::string, Meta>> meta;   // file order
    std::map<std::string, size_t> meta_ix;
    std::vector<TensorInfo> tensors;
    std::map<std::string, size_t> tensor_ix;
    uint64_t data_start = 0;
};

namespace {

int parse_into(fhip_gguf& g) {
    Window c{g.bytes, g.bytes + g.len};
    const uint32_t magic = c.scalar<uint32_t>();
    if (c.bad || magic != 0x46554747u) return fhip::set_error(FHIP_ERR_FORMAT, "not a GGUF file");   // "GGUF" little endian
    g.version = c.scalar<uint32_t>();
    const uint64_t n_tensors = c.scalar<uint64_t>(), n_meta = c.scalar<uint64_t>();
    for (uint64_t k = 0; k < n_meta && !c.bad; k++) {
        std::string key = c.text();
        const uint32_t ty = c.scalar<uint32_t>();
        Meta m = read_value(c, ty);
        auto it = g.meta_ix.find(key);
        if (it != g.meta_ix.end()) g.meta[it->second].second = std::move(m);   // a repeated key keeps the last value (HashMap::insert)
        else { g.meta_ix[key] = g.meta.size(); g.meta.emplace_back(std::move(key), std::move(m)); }
    }
    for (uint64_t k = 0; k < n_tensors && !c.bad; k++) {
        TensorInfo t;
        t.name = c.text();
        const uint32_t nd = c.scalar<uint32_t>();
        if ((uint64_t)nd * 8 > c.left()) { c.bad = true; break; }
        for (uint32_t d = 0; d < nd; d++) t.dims.push_back(c.scalar<uint64_t>());
        t.ggml_type = c.scalar<uint32_t>();
        t.offset = c.scalar<uint64_t>();
        g.tensors.push_back(std::move(t));
    }
    if (c.bad) return fhip::set_error(FHIP_ERR_FORMAT, "GGUF header truncated or malformed");
    for (size_t i = 0; i < g.tensors.size(); i++) g.tensor_ix.emplace(g.tensors[i].name, i);   // first of a repeated name, as `find`
    uint64_t align = 32;
    auto al = g.meta_ix.find("general.alignment");
    if (al != g.meta_ix.end() && g.meta[al->second].second.kind == K_U) align = g.meta[al->second].second.u;
    if (align == 0) return fhip::set_error(FHIP_ERR_FORMAT, "GGUF general.alignment is 0");
    g.data_start = ((size_t)(c.at - g.bytes) + align - 1) / align * align;
    const uint64_t data_len = g.len > g.data_start ? g.len - g.data_start : 0;
    const std::string why = check_declared_strides(g.tensors, data_len, align);
    if (!why.empty()) return fhip::set_error(FHIP_ERR_FORMAT, "%s", why.c_str());
    return FHIP_OK;
}

const Meta* find_meta(const fhip_gguf* g, const char* key) {
    if (!g || !key) return nullptr;
    auto it = g->meta_ix.find(key);
    return it == g->meta_ix.end() ? nullptr : &g->meta[it->second].second;
}

}  // namespace

extern "C" {

int fhip_gguf_parse(const uint8_t* bytes, size_t n, fhip_gguf** out) {
    if (!out) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_parse: NULL output");
    *out = nullptr;
    if (!bytes && n) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_parse: NULL bytes");
    fhip_gguf* g = new fhip_gguf;
    g->bytes = bytes;
    g->len = n;
    const int rc = parse_into(*g);
    if (rc) { delete g; return rc; }
    *out = g;
    return FHIP_OK;
}

int fhip_gguf_open(const char* path, fhip_gguf** out) {
    if (!out) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_open: NULL output");
    *out = nullptr;
    if (!path) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_open: NULL path");
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_open: cannot open '%s': %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) { const int e = errno; close(fd); return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_open: fstat '%s': %s", path, strerror(e)); }
    void* map = nullptr;
    if (st.st_size > 0) {
        map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
        if (map == MAP_FAILED) { const int e = errno; close(fd); return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_open: mmap '%s': %s", path, strerror(e)); }
    }
    close(fd);
    fhip_gguf* g = new fhip_gguf;
    g->bytes = (const uint8_t*)map;
    g->len = (size_t)st.st_size;
    g->map = map;
    g->map_len = (size_t)st.st_size;
    const int rc = parse_into(*g);
    if (rc) { fhip_gguf_close(g); return rc; }
    *out = g;
    return FHIP_OK;
}

void fhip_gguf_close(fhip_gguf* g) {
    if (!g) return;
    if (g->map) munmap(g->map, g->map_len);
    delete g;
}

size_t fhip_gguf_n_tensors(const fhip_gguf* g) { return g ? g->tensors.size() : 0; }
uint64_t fhip_gguf_data_start(const fhip_gguf* g) { return g ? g->data_start : 0; }
uint32_t fhip_gguf_version(const fhip_gguf* g) { return g ? g->version : 0; }

int fhip_gguf_tensor(const fhip_gguf* g, size_t i, const char** name, uint32_t* n_dims, const uint64_t** dims, uint32_t* ggml_type,
                     uint64_t* offset) {
    if (!g || i >= g->tensors.size()) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_tensor: index out of range");
    const TensorInfo& t = g->tensors[i];
    if (name) *name = t.name.c_str();
    if (n_dims) *n_dims = (uint32_t)t.dims.size();
    if (dims) *dims = t.dims.data();
    if (ggml_type) *ggml_type = t.ggml_type;
    if (offset) *offset = t.offset;
    return FHIP_OK;
}

long fhip_gguf_find(const fhip_gguf* g, const char* name) {
    if (!g || !name) return -1;
    auto it = g->tensor_ix.find(name);
    return it == g->tensor_ix.end() ? -1 : (long)it->second;
}

int fhip_gguf_raw(const fhip_gguf* g, const char* name, const uint8_t** bytes, size_t* nbytes) {
    if (!g || !name || !bytes || !nbytes) return fhip::set_error(FHIP_ERR_ARG, "fhip_gguf_raw: NULL argument");
    const long i = fhip_gguf_find(g, name);
    if (i < 0) return fhip::set_error(FHIP_ERR_FORMAT, "no tensor '%s'", name);
    const TensorInfo& t = g->tensors[(size_t)i];
    uint64_t sz;
    if (!type_size_all(t.ggml_type, numel(t), &sz)) return fhip::set_error(FHIP_ERR_UNSUPPORTED_TYPE, "unsupported ggml type %u", t.ggml_type);
    const uint64_t start = g->data_start + t.offset;
    if (start > g->len || sz > g->len - start)
        return fhip::set_error(FHIP_ERR_FORMAT, "tensor '%s' extends past the end of the file (%llu + %llu > %zu)", name,
                               (unsigned long long)start, (unsigned long long)sz, g->len);
    *bytes = g->bytes + start;
    *nbytes = (size_t)sz;
    return FHIP_OK;
}

size_t fhip_gguf_n_meta(const fhip_gguf* g) { return g ? g->meta.size() : 0; }
const char* fhip_gguf_meta_key(const fhip_gguf* g, size_t i) { return g && i < g->meta.size() ? g->meta[i].first.c_str() : nullptr; }

int fhip_gguf_meta_kind(const fhip_gguf* g, const char* key, size_t* arr_len) {
    const Meta* m = find_meta(g, key);
    if (!m) return -1;
    if (arr_len) *arr_len = m->kind == K_ARR ? m->a.size() : 0;
    return m->kind;
}

// element j of an array value, or the value itself when j == (size_t)-1
static const Meta* pick(const fhip_gguf* g, const char* key, size_t j) {
    const Meta* m = find_meta(g, key);
    if (!m) return nullptr;
    if (j == (size_t)-1) return m;
    return m->kind == K_ARR && j < m->a.size() ? &m->a[j] : nullptr;
}

int fhip_gguf_meta_u64(const fhip_gguf* g, const char* key, size_t j, uint64_t* out) {
    const Meta* m = pick(g, key, j);
    if (!m || !out || (m->kind != K_U && m->kind != K_BOOL)) return fhip::set_error(FHIP_ERR_FORMAT, "metadata '%s' is absent or not unsigned", key ? key : "");
    *out = m->u;
    return FHIP_OK;
}
int fhip_gguf_meta_i64(const fhip_gguf* g, const char* key, size_t j, int64_t* out) {
    const Meta* m = pick(g, key, j);
    if (!m || !out || m->kind != K_I) return fhip::set_error(FHIP_ERR_FORMAT, "metadata '%s' is absent or not signed", key ? key : "");
    *out = m->i;
    return FHIP_OK;
}
int fhip_gguf_meta_f64(const fhip_gguf* g, const char* key, size_t j, double* out) {
    const Meta* m = pick(g, key, j);
    if (!m || !out || m->kind != K_F) return fhip::set_error(FHIP_ERR_FORMAT, "metadata '%s' is absent or not a float", key ? key : "");
    *out = m->f;
    return FHIP_OK;
}
int fhip_gguf_meta_str(const fhip_gguf* g, const char* key, size_t j, const char** s, size_t* len) {
    const Meta* m = pick(g, key, j);
    if (!m || !s || !len || m->kind != K_STR) return fhip::set_error(FHIP_ERR_FORMAT, "metadata '%s' is absent or not a string", key ? key : "");
    *s = m->s.data();
    *len = m->s.size();
    return FHIP_OK;
}

int fhip_weight_from_gguf(const fhip_gguf* g, const char* name, fhip_weight** out) {
    if (!out) return fhip::set_error(FHIP_ERR_ARG, "fhip_weight_from_gguf: NULL output");
    *out = nullptr;
    const uint8_t* bytes;
    size_t nbytes;
    int rc = fhip_gguf_raw(g, name, &bytes, &nbytes);
    if (rc) return rc;
    const TensorInfo& t = g->tensors[(size_t)fhip_gguf_find(g, name)];
    if (t.dims.size() < 2) return fhip::set_error(FHIP_ERR_SHAPE, "tensor '%s' has %zu dims; a weight needs [in, out(, experts)]", name, t.dims.size());
    // GGUF lists the fastest dimension first: dims[0] = in (cols); the others multiply into rows (an expert slab
    // [in, rows per expert, n_expert] is expert-major, which is what the "_id" entry points index)
    uint64_t rows = 1;
    for (size_t d = 1; d < t.dims.size(); d++) rows *= t.dims[d];
    return fhip_weight_create(t.ggml_type, bytes, nbytes, (size_t)rows, (size_t)t.dims[0], out);
}

int fhip_weight_from_gguf_cat(const fhip_gguf* g, const char* const* names, size_t n_names, fhip_weight** out) {
    if (!out) return fhip::set_error(FHIP_ERR_ARG, "fhip_weight_from_gguf_cat: NULL output");
    *out = nullptr;
    if (!g || !names || n_names == 0) return fhip::set_error(FHIP_ERR_ARG, "fhip_weight_from_gguf_cat: nothing to concatenate");
    // crates/ferric-llama/src/qwen35.rs:381-390: one format, one input width, the output widths add up
    std::vector<const uint8_t*> parts(n_names);
    std::vector<size_t> sizes(n_names);
    uint32_t ty = 0;
    uint64_t inn = 0, rows = 0;
    for (size_t i = 0; i < n_names; i++) {
        const char* name = names[i];
        if (!name) return fhip::set_error(FHIP_ERR_ARG, "fhip_weight_from_gguf_cat: NULL name");
        const int64_t at = fhip_gguf_find(g, name);
        if (at < 0) return fhip::set_error(FHIP_ERR_FORMAT, "no tensor '%s'", name);
        const TensorInfo& t = g->tensors[(size_t)at];
        if (t.dims.size() < 2) return fhip::set_error(FHIP_ERR_SHAPE, "tensor '%s' has %zu dims; a weight needs [in, out]", name, t.dims.size());
        if (i == 0) { ty = t.ggml_type; inn = t.dims[0]; }
        if (t.ggml_type != ty) return fhip::set_error(FHIP_ERR_FORMAT, "%s: mixed quant formats in one fused matmul", name);
        if (t.dims[0] != inn) return fhip::set_error(FHIP_ERR_FORMAT, "%s: input dim differs", name);
        rows += t.dims[1];
        int rc = fhip_gguf_raw(g, name, &parts[i], &sizes[i]);
        if (rc) return rc;
    }
    return fhip_weight_create_parts(ty, parts.data(), sizes.data(), n_names, (size_t)rows, (size_t)inn, out);
}

}  // extern "C"
