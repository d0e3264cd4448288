// Weight bundles: "<model>.bin" (tensors back to back in sorted-name order, no padding)
// plus "<model>.meta.json" (per tensor: offset, shape, dtype, num_elements, size_bytes).
// Layout authority: scripts/convert_hf_to_bin.py:149-170 (fp16 bundles),
// LF/scripts/quantize_weights.py:141-175 (int8: "<name>" int8 [N,K] followed by
// "<name>.scale" fp16 [N]) and LF/scripts/quantize_q4.py:168-185 ("q4_packed" [N,K/2]
// followed by "<name>.scale" fp16 [N,K/32]).  Host side mirrors Weights::load /
// get_buffer (QW/src/weights.cpp:165-293): the .bin is mmap-ed read-only and device
// copies are made per tensor, each in its own allocation (so every tensor is aligned).
#include "../../include/mi_linear.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#define BUNDLE_ERROR(fmt, ...) \
    std::fprintf(stderr, "ERROR: " fmt " (%s:%d)\n", ##__VA_ARGS__, __FILE__, __LINE__)

namespace {

struct Tensor {
    size_t offset = 0, size_bytes = 0, num_elements = 0;
    std::vector<int64_t> shape;
    std::string dtype;
    void* dev = nullptr;
    bool registered = false;
};

struct Bundle {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t map_size = 0;
    std::map<std::string, Tensor> tensors;   // std::map iterates in sorted-name order
    std::vector<const std::string*> order;
};

// ---- a small JSON reader: enough for meta.json (objects, arrays, strings, numbers,
// true/false/null), with the usual escapes ------------------------------------------
struct Json {
    enum Type { Null, Bool, Num, Str, Arr, Obj } type = Null;
    double num = 0;
    bool b = false;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;
    const Json* get(const char* key) const {
        for (auto& kv : obj) if (kv.first == key) return &kv.second;
        return nullptr;
    }
};

struct Parser {
    const char* p;
    const char* end;
    bool ok = true;
    void ws() { while (p < end && std::isspace(static_cast<unsigned char>(*p))) ++p; }
    bool eat(char c) { ws(); if (p < end && *p == c) { ++p; return true; } return false; }
    std::string string() {
        std::string s;
        if (!eat('"')) { ok = false; return s; }
        while (p < end && *p != '"') {
            if (*p == '\\' && p + 1 < end) {
                ++p;
                switch (*p) {
                    case 'n': s += '\n'; break;
                    case 't': s += '\t'; break;
                    case 'r': s += '\r'; break;
                    case 'b': s += '\b'; break;
                    case 'f': s += '\f'; break;
                    case 'u': {
                        if (p + 4 < end) {
                            unsigned cp = static_cast<unsigned>(std::strtoul(std::string(p + 1, p + 5).c_str(), nullptr, 16));
                            if (cp < 0x80) s += static_cast<char>(cp);
                            else if (cp < 0x800) { s += static_cast<char>(0xC0 | (cp >> 6)); s += static_cast<char>(0x80 | (cp & 0x3F)); }
                            else { s += static_cast<char>(0xE0 | (cp >> 12)); s += static_cast<char>(0x80 | ((cp >> 6) & 0x3F)); s += static_cast<char>(0x80 | (cp & 0x3F)); }
                            p += 4;
                        } else ok = false;
                        break;
                    }
                    default: s += *p;
                }
                ++p;
            } else s += *p++;
        }
        if (p >= end) { ok = false; return s; }
        ++p;
        return s;
    }
    Json value() {
        Json v;
        ws();
        if (p >= end) { ok = false; return v; }
        if (*p == '{') {
            ++p; v.type = Json::Obj;
            if (eat('}')) return v;
            do {
                std::string k = string();
                if (!ok || !eat(':')) { ok = false; return v; }
                v.obj.emplace_back(std::move(k), value());
                if (!ok) return v;
            } while (eat(','));
            if (!eat('}')) ok = false;
        } else if (*p == '[') {
            ++p; v.type = Json::Arr;
            if (eat(']')) return v;
            do { v.arr.push_back(value()); if (!ok) return v; } while (eat(','));
            if (!eat(']')) ok = false;
        } else if (*p == '"') {
            v.type = Json::Str; v.str = string();
        } else if (!std::strncmp(p, "true", std::min<size_t>(4, end - p))) { v.type = Json::Bool; v.b = true; p += 4; }
        else if (!std::strncmp(p, "false", std::min<size_t>(5, end - p))) { v.type = Json::Bool; p += 5; }
        else if (!std::strncmp(p, "null", std::min<size_t>(4, end - p))) { p += 4; }
        else {
            char* e = nullptr;
            v.type = Json::Num; v.num = std::strtod(p, &e);
            if (e == p) ok = false;
            p = e;
        }
        return v;
    }
};

size_t bytes_per_element(const std::string& dtype) {      // LF/src/weights.cpp:143-148
    if (dtype == "float16" || dtype == "bfloat16") return 2;
    if (dtype == "int8" || dtype == "q4_packed") return 1;
    return 4;
}

}  // namespace

extern "C" {

void* mi_bundle_open(const char* bin_path, const char* meta_path) {
    if (!bin_path || !meta_path) { BUNDLE_ERROR("bundle: null path"); return nullptr; }
    auto* b = new Bundle;
    b->fd = open(bin_path, O_RDONLY);
    struct stat st;
    if (b->fd < 0 || fstat(b->fd, &st) != 0 || st.st_size <= 0) {
        BUNDLE_ERROR("weights: failed to open %s for mmap", bin_path);
        mi_bundle_close(b);
        return nullptr;
    }
    b->map_size = static_cast<size_t>(st.st_size);
    void* m = mmap(nullptr, b->map_size, PROT_READ, MAP_PRIVATE, b->fd, 0);
    if (m == MAP_FAILED) {
        BUNDLE_ERROR("weights: mmap of %s failed", bin_path);
        mi_bundle_close(b);
        return nullptr;
    }
    b->map = static_cast<const uint8_t*>(m);

    std::ifstream f(meta_path);
    if (!f.is_open()) {
        BUNDLE_ERROR("Failed to open metadata: %s", meta_path);
        mi_bundle_close(b);
        return nullptr;
    }
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str();
    Parser ps{text.data(), text.data() + text.size()};
    const Json root = ps.value();
    const Json* tensors = ps.ok ? root.get("tensors") : nullptr;
    if (!tensors || tensors->type != Json::Obj) {
        BUNDLE_ERROR("Could not parse weight metadata from %s", meta_path);
        mi_bundle_close(b);
        return nullptr;
    }
    for (auto& kv : tensors->obj) {
        const Json& t = kv.second;
        const Json *off = t.get("offset"), *sz = t.get("size_bytes"), *shape = t.get("shape"), *dt = t.get("dtype");
        if (!off || !sz || !shape || shape->type != Json::Arr) {
            BUNDLE_ERROR("meta: tensor '%s' lacks offset/size_bytes/shape", kv.first.c_str());
            mi_bundle_close(b);
            return nullptr;
        }
        Tensor tm;
        tm.offset = static_cast<size_t>(off->num);
        tm.size_bytes = static_cast<size_t>(sz->num);
        tm.dtype = dt && dt->type == Json::Str ? dt->str : "float32";
        tm.num_elements = tm.size_bytes / bytes_per_element(tm.dtype);
        for (auto& d : shape->arr) tm.shape.push_back(static_cast<int64_t>(d.num));
        if (tm.offset + tm.size_bytes > b->map_size) {
            BUNDLE_ERROR("meta: tensor '%s' exceeds file bounds (%zu + %zu > %zu)", kv.first.c_str(),
                         tm.offset, tm.size_bytes, b->map_size);
            mi_bundle_close(b);
            return nullptr;
        }
        size_t prod = 1;
        for (auto d : tm.shape) prod *= static_cast<size_t>(d);
        if (prod != tm.num_elements) {
            BUNDLE_ERROR("meta: tensor '%s' shape product %zu != %zu elements", kv.first.c_str(), prod,
                         tm.num_elements);
            mi_bundle_close(b);
            return nullptr;
        }
        b->tensors[kv.first] = std::move(tm);
    }
    for (auto& kv : b->tensors) b->order.push_back(&kv.first);
    return b;
}

void mi_bundle_close(void* h) {
    auto* b = static_cast<Bundle*>(h);
    if (!b) return;
    // registry entries are keyed by the device pointer: they go before the allocation does, so
    // that a later allocation at the same address is not mistaken for this bundle's weight
    for (auto& kv : b->tensors) {
        if (kv.second.registered) mi_unregister_weight(kv.second.dev);
        if (kv.second.dev) mi_free(kv.second.dev);
    }
    if (b->map) munmap(const_cast<uint8_t*>(b->map), b->map_size);
    if (b->fd >= 0) close(b->fd);
    delete b;
}

int mi_bundle_count(void* h) { return h ? static_cast<int>(static_cast<Bundle*>(h)->order.size()) : 0; }

const char* mi_bundle_name(void* h, int i) {
    auto* b = static_cast<Bundle*>(h);
    if (!b || i < 0 || i >= static_cast<int>(b->order.size())) return nullptr;
    return b->order[i]->c_str();
}

int mi_bundle_tensor(void* h, const char* name, const void** host_ptr, size_t* size_bytes,
                     const char** dtype, int* ndim, int64_t shape[4]) {
    auto* b = static_cast<Bundle*>(h);
    if (!b || !name) return 0;
    auto it = b->tensors.find(name);
    if (it == b->tensors.end()) return 0;
    const Tensor& t = it->second;
    if (host_ptr) *host_ptr = b->map + t.offset;
    if (size_bytes) *size_bytes = t.size_bytes;
    if (dtype) *dtype = t.dtype.c_str();
    if (ndim) *ndim = static_cast<int>(t.shape.size());
    if (shape) for (size_t i = 0; i < 4; ++i) shape[i] = i < t.shape.size() ? t.shape[i] : 0;
    return 1;
}

int mi_bundle_upload(void* h) {
    auto* b = static_cast<Bundle*>(h);
    if (!b) return -1;
    for (auto& kv : b->tensors) {
        Tensor& t = kv.second;
        if (t.dev) continue;
        t.dev = mi_malloc(t.size_bytes);
        if (!t.dev || !mi_memcpy_h2d(t.dev, b->map + t.offset, t.size_bytes, nullptr)) {
            BUNDLE_ERROR("Failed to create buffer for %s", kv.first.c_str());
            return -1;
        }
    }
    // LF/src/main.cpp:527-566: every int8 / q4_packed 2-D tensor with a scale sibling.
    // LFM2-VL bundles spell the sibling ".scales" (LV/scripts/quantize_int8.py:91-97).
    int registered = 0;
    for (auto& kv : b->tensors) {
        Tensor& t = kv.second;
        if (t.registered) { ++registered; continue; }
        if ((t.dtype != "int8" && t.dtype != "q4_packed") || t.shape.size() != 2) continue;
        auto sit = b->tensors.find(kv.first + ".scale");
        if (sit == b->tensors.end()) sit = b->tensors.find(kv.first + ".scales");
        if (sit == b->tensors.end()) continue;
        const Tensor& s = sit->second;
        int ok;
        if (t.dtype == "int8") {
            ok = mi_register_int8_weight(t.dev, s.dev, static_cast<int>(t.shape[0]), static_cast<int>(t.shape[1]));
        } else {
            if (s.shape.size() != 2) continue;
            ok = mi_register_q4_weight(t.dev, s.dev, static_cast<int>(t.shape[0]), static_cast<int>(s.shape[1] * 32));
        }
        t.registered = ok != 0;
        registered += ok;
    }
    return registered;
}

void* mi_bundle_device_ptr(void* h, const char* name) {
    auto* b = static_cast<Bundle*>(h);
    if (!b || !name) return nullptr;
    auto it = b->tensors.find(name);
    return it == b->tensors.end() ? nullptr : it->second.dev;
}

}  // extern "C"
