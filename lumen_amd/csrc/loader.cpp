// ModelLoader::load_llama_weights, src/loader.rs:10-80: memory-map a
// .safetensors file and copy every parameter of the model that the file holds
// into the model, F32 as is, BF16 widened (or kept as bf16 bits when the model
// stores bf16); parameters the file lacks are counted and left as they are
// (the reference prints a warning, :69-74), any other dtype is an error (:67).
//
// The container format is the public safetensors layout: 8 bytes little-endian
// header length N, N bytes of JSON {"name": {"dtype": "...", "shape": [...],
// "data_offsets": [begin, end]}, ..., "__metadata__": {...}}, then the raw
// tensor bytes, offsets relative to the end of the header.  The reference
// reads it through the `safetensors` crate; this is a stand-alone reader.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdint>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/lumen_hip.h"

void lumen_set_error(const char *fmt, ...);
// names of the model's parameters in the order of LlamaModel::named_parameters and their shapes
int lumen_llama_param_list(const lumen_llama *m, std::vector<std::string> &names, std::vector<std::vector<int64_t>> &shapes);

namespace {

struct Entry {
    std::string dtype;
    std::vector<int64_t> shape;
    uint64_t begin = 0, end = 0;
};

// Minimal JSON reader for the header: objects, arrays, strings, numbers, true/false/null.
struct Json {
    const char *p, *e;
    bool fail = false;
    void ws() {
        while (p < e && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
    }
    bool eat(char c) {
        ws();
        if (p < e && *p == c) {
            ++p;
            return true;
        }
        return false;
    }
    std::string str() {
        std::string s;
        ws();
        if (p >= e || *p != '"') {
            fail = true;
            return s;
        }
        ++p;
        while (p < e && *p != '"') {
            if (*p == '\\' && p + 1 < e) {
                ++p;
                switch (*p) {
                    case 'n': s += '\n'; break;
                    case 't': s += '\t'; break;
                    case 'r': s += '\r'; break;
                    case 'b': s += '\b'; break;
                    case 'f': s += '\f'; break;
                    case 'u':  // keep the escape as written: parameter names are plain ASCII
                        s += "\\u";
                        break;
                    default: s += *p;
                }
                ++p;
            } else {
                s += *p++;
            }
        }
        if (p >= e) {
            fail = true;
            return s;
        }
        ++p;
        return s;
    }
    bool number(uint64_t &v) {
        ws();
        const char *s = p;
        v = 0;
        while (p < e && *p >= '0' && *p <= '9') v = v * 10 + (uint64_t)(*p++ - '0');
        return p > s;
    }
    void skip(int depth = 0) {  // any value; nesting beyond 64 levels is refused (no file of this format has it)
        ws();
        if (p >= e || depth > 64) {
            fail = true;
            return;
        }
        if (*p == '"') {
            str();
        } else if (*p == '{') {
            ++p;
            if (eat('}')) return;
            do {
                str();
                if (!eat(':')) {
                    fail = true;
                    return;
                }
                skip(depth + 1);
            } while (!fail && eat(','));
            if (!eat('}')) fail = true;
        } else if (*p == '[') {
            ++p;
            if (eat(']')) return;
            do skip(depth + 1);
            while (!fail && eat(','));
            if (!eat(']')) fail = true;
        } else {
            while (p < e && *p != ',' && *p != '}' && *p != ']') ++p;
        }
    }
};

bool parse_header(const char *h, size_t n, std::map<std::string, Entry> &out) {
    Json j{h, h + n};
    if (!j.eat('{')) return false;
    if (j.eat('}')) return true;
    do {
        const std::string name = j.str();
        if (j.fail || !j.eat(':')) return false;
        if (name == "__metadata__") {
            j.skip();
            if (j.fail) return false;
            continue;
        }
        Entry en;
        if (!j.eat('{')) return false;
        do {
            const std::string key = j.str();
            if (j.fail || !j.eat(':')) return false;
            if (key == "dtype") {
                en.dtype = j.str();
            } else if (key == "shape") {
                if (!j.eat('[')) return false;
                if (!j.eat(']')) {
                    do {
                        uint64_t v;
                        if (!j.number(v)) return false;
                        en.shape.push_back((int64_t)v);
                    } while (j.eat(','));
                    if (!j.eat(']')) return false;
                }
            } else if (key == "data_offsets") {
                if (!j.eat('[') || !j.number(en.begin) || !j.eat(',') || !j.number(en.end) || !j.eat(']')) return false;
            } else {
                j.skip();
            }
            if (j.fail) return false;
        } while (j.eat(','));
        if (!j.eat('}')) return false;
        out[name] = en;
    } while (j.eat(','));
    return j.eat('}');
}

struct Mapping {
    void *p = MAP_FAILED;
    size_t n = 0;
    int fd = -1;
    ~Mapping() {
        if (p != MAP_FAILED) munmap(p, n);
        if (fd >= 0) close(fd);
    }
};

}  // namespace

// Opens and parses a file; on success `map` holds the mapping, `entries` the header, `data` the
// first byte after the header.
static int open_safetensors(const char *path, Mapping &map, std::map<std::string, Entry> &entries,
                            const unsigned char *&data, uint64_t &data_len) {
    map.fd = open(path, O_RDONLY);
    struct stat st;
    if (map.fd < 0 || fstat(map.fd, &st) != 0) {
        lumen_set_error("cannot open %s: %s", path, strerror(errno));
        return LUMEN_ERR_INVALID;
    }
    map.n = (size_t)st.st_size;
    if (map.n < 8) {
        lumen_set_error("%s: too short for a safetensors header", path);
        return LUMEN_ERR_INVALID;
    }
    map.p = mmap(nullptr, map.n, PROT_READ, MAP_PRIVATE, map.fd, 0);
    if (map.p == MAP_FAILED) {
        lumen_set_error("cannot map %s: %s", path, strerror(errno));
        return LUMEN_ERR_INVALID;
    }
    const unsigned char *base = (const unsigned char *)map.p;
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | base[i];
    if (hlen > map.n - 8) {
        lumen_set_error("%s: header length %llu exceeds the file", path, (unsigned long long)hlen);
        return LUMEN_ERR_INVALID;
    }
    if (!parse_header((const char *)base + 8, (size_t)hlen, entries)) {
        lumen_set_error("%s: malformed safetensors header", path);
        return LUMEN_ERR_INVALID;
    }
    data = base + 8 + hlen;
    data_len = map.n - 8 - hlen;
    return LUMEN_OK;
}

extern "C" int lumen_safetensors_find(const char *path, const char *name, int *dtype_out, int64_t *shape_out,
                                      int *ndim_inout, uint64_t *begin_out, uint64_t *end_out) {
    if (!path || !name || !dtype_out || !shape_out || !ndim_inout || !begin_out || !end_out) {
        lumen_set_error("safetensors_find: null argument");
        return LUMEN_ERR_INVALID;
    }
    Mapping map;
    std::map<std::string, Entry> entries;
    const unsigned char *data = nullptr;
    uint64_t data_len = 0;
    const int rc = open_safetensors(path, map, entries, data, data_len);
    if (rc != LUMEN_OK) return rc;
    auto it = entries.find(name);
    if (it == entries.end()) {
        lumen_set_error("Parameter %s not found in safetensors file", name);
        return LUMEN_ERR_INVALID;
    }
    const Entry &en = it->second;
    if ((int)en.shape.size() > *ndim_inout) {
        lumen_set_error("safetensors_find: %s has %zu dimensions, room for %d", name, en.shape.size(), *ndim_inout);
        return LUMEN_ERR_SHAPE;
    }
    *dtype_out = en.dtype == "F32" ? LUMEN_DTYPE_F32 : en.dtype == "BF16" ? LUMEN_DTYPE_BF16 : -1;
    *ndim_inout = (int)en.shape.size();
    for (size_t i = 0; i < en.shape.size(); ++i) shape_out[i] = en.shape[i];
    *begin_out = en.begin;
    *end_out = en.end;
    return LUMEN_OK;
}

extern "C" int lumen_llama_load_safetensors(lumen_llama *m, const char *path, int *n_loaded_out, int *n_missing_out) {
    if (n_loaded_out) *n_loaded_out = 0;
    if (n_missing_out) *n_missing_out = 0;
    if (!m || !path) {
        lumen_set_error("llama_load_safetensors: null argument");
        return LUMEN_ERR_INVALID;
    }
    Mapping map;
    std::map<std::string, Entry> entries;
    const unsigned char *data = nullptr;
    uint64_t data_len = 0;
    int rc = open_safetensors(path, map, entries, data, data_len);
    if (rc != LUMEN_OK) return rc;

    std::vector<std::string> names;
    std::vector<std::vector<int64_t>> shapes;
    rc = lumen_llama_param_list(m, names, shapes);
    if (rc != LUMEN_OK) return rc;
    int loaded = 0, missing = 0;
    for (size_t i = 0; i < names.size(); ++i) {
        auto it = entries.find(names[i]);
        if (it == entries.end()) {  // loader.rs:69-74: a warning, not an error
            ++missing;
            continue;
        }
        const Entry &en = it->second;
        int dtype;
        size_t esz;
        if (en.dtype == "F32") {
            dtype = LUMEN_DTYPE_F32;
            esz = 4;
        } else if (en.dtype == "BF16") {
            dtype = LUMEN_DTYPE_BF16;
            esz = 2;
        } else {  // loader.rs:67
            lumen_set_error("Unsupported dtype: %s for %s", en.dtype.c_str(), names[i].c_str());
            return LUMEN_ERR_INVALID;
        }
        if (en.end < en.begin || en.end > data_len) {
            lumen_set_error("%s: data offsets of %s outside the file", path, names[i].c_str());
            return LUMEN_ERR_INVALID;
        }
        // the reference reshapes the file's elements to the parameter's shape and fails when the
        // counts differ (Array::from_shape_vec, loader.rs:44-46, 60-62)
        uint64_t want = 1;
        for (int64_t d : shapes[i]) want *= (uint64_t)d;
        if ((en.end - en.begin) / esz != want || (en.end - en.begin) % esz) {
            lumen_set_error("Shape mismatch for %s: %llu elements in the file, %llu in the model", names[i].c_str(),
                            (unsigned long long)((en.end - en.begin) / esz), (unsigned long long)want);
            return LUMEN_ERR_SHAPE;
        }
        rc = lumen_llama_set_param(m, names[i].c_str(), data + en.begin, dtype, shapes[i].data(), (int)shapes[i].size());
        if (rc != LUMEN_OK) return rc;
        ++loaded;
    }
    if (n_loaded_out) *n_loaded_out = loaded;
    if (n_missing_out) *n_missing_out = missing;
    return LUMEN_OK;
}
