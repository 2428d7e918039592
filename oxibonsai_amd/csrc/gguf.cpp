// gguf.cpp — GGUF reader (host only).  See gguf.h for the format summary and the reference files it follows.
#include "gguf.h"

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>

namespace oxb {

namespace {

constexpr uint32_t kMagic = 0x46554747u;            // "GGUF", header.rs:8
constexpr uint64_t kMaxString = 256ull << 20;       // tensor_info.rs MAX_STRING_LEN
constexpr uint32_t kMaxDims = 1024;                 // tensor_info.rs MAX_TENSOR_DIMS

// Bounds-checked little-endian cursor over the mapping.
struct Cursor {
    const uint8_t* p;
    size_t size, pos;
    bool ok = true;
    size_t fail_at = 0;

    bool need(size_t n) {
        if (!ok) return false;
        if (n > size - pos) {
            ok = false;
            fail_at = pos;
            return false;
        }
        return true;
    }
    template <typename T>
    T get() {
        T v{};
        if (need(sizeof(T))) {
            memcpy(&v, p + pos, sizeof(T));  // the build targets little-endian hosts only
            pos += sizeof(T);
        }
        return v;
    }
    std::string str() {
        const uint64_t len = get<uint64_t>();
        if (!ok) return {};
        if (len > kMaxString || !need((size_t)len)) {
            if (ok) ok = false, fail_at = pos;
            return {};
        }
        std::string s(reinterpret_cast<const char*>(p + pos), (size_t)len);
        pos += (size_t)len;
        return s;
    }
};

size_t scalar_size(uint32_t type) {
    switch (type) {
        case 0: case 1: case 7: return 1;  // u8, i8, bool
        case 2: case 3: return 2;          // u16, i16
        case 4: case 5: case 6: return 4;  // u32, i32, f32
        case 10: case 11: case 12: return 8;  // u64, i64, f64
        default: return 0;
    }
}

bool read_value(Cursor& c, uint32_t type, GgufValue* v, int depth) {
    v->type = type;
    switch (type) {
        case 0: v->u = c.get<uint8_t>(); break;
        case 1: v->i = c.get<int8_t>(); break;
        case 2: v->u = c.get<uint16_t>(); break;
        case 3: v->i = c.get<int16_t>(); break;
        case 4: v->u = c.get<uint32_t>(); break;
        case 5: v->i = c.get<int32_t>(); break;
        case 6: v->f = c.get<float>(); break;
        case 7: v->u = c.get<uint8_t>() != 0; break;
        case 8: v->s = c.str(); break;
        case 10: v->u = c.get<uint64_t>(); break;
        case 11: v->i = c.get<int64_t>(); break;
        case 12: v->f = c.get<double>(); break;
        case 9: {  // array: element type, count, elements (skipped: this tier reads no array-valued key)
            v->elem_type = c.get<uint32_t>();
            v->count = c.get<uint64_t>();
            if (!c.ok) return false;
            const size_t es = scalar_size(v->elem_type);
            if (es) {
                if (v->count > (c.size - c.pos) / es) {
                    c.ok = false, c.fail_at = c.pos;
                    return false;
                }
                c.pos += (size_t)v->count * es;
            } else if (v->elem_type == 8) {
                for (uint64_t i = 0; i < v->count && c.ok; i++) (void)c.str();
            } else if (v->elem_type == 9 && depth < 4) {
                for (uint64_t i = 0; i < v->count && c.ok; i++) {
                    GgufValue inner;
                    if (!read_value(c, 9, &inner, depth + 1)) return false;
                }
            } else {
                return false;
            }
            break;
        }
        default: return false;  // unknown value type: the rest of the file cannot be located
    }
    return c.ok;
}

}  // namespace

uint64_t gguf_tensor_bytes(uint32_t type, uint64_t elements) {
    switch (type) {
        case GGUF_F32: return elements * 4;
        case GGUF_F16: return elements * 2;
        case GGUF_Q1_0_G128: return (elements + 127) / 128 * 18;
        case GGUF_TQ2_0_G128: return (elements + 127) / 128 * 34;
        default: return 0;
    }
}

GgufFile::~GgufFile() {
    if (base_) munmap(const_cast<uint8_t*>(base_), size_);
    if (fd_ >= 0) close(fd_);
}

bool GgufFile::open(const char* path, std::string* err) {
    char msg[256];
    auto failf = [&](const char* m) {
        *err = m;
        return false;
    };
    if (!path) return failf("null path");
    fd_ = ::open(path, O_RDONLY);
    if (fd_ < 0) {
        snprintf(msg, sizeof msg, "cannot open %s: %s", path, strerror(errno));
        return failf(msg);
    }
    struct stat stt;
    if (fstat(fd_, &stt) != 0 || stt.st_size <= 0) {
        snprintf(msg, sizeof msg, "unexpected end of file at offset 0 (%s is empty or unreadable)", path);
        return failf(msg);
    }
    size_ = (size_t)stt.st_size;
    void* mp = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (mp == MAP_FAILED) {
        snprintf(msg, sizeof msg, "cannot map %s: %s", path, strerror(errno));
        return failf(msg);
    }
    base_ = static_cast<const uint8_t*>(mp);

    Cursor c{base_, size_, 0};
    const uint32_t magic = c.get<uint32_t>();
    if (!c.ok) return failf("unexpected end of file at offset 0");
    if (magic != kMagic) {
        snprintf(msg, sizeof msg, "invalid GGUF magic 0x%08X", magic);
        return failf(msg);
    }
    version = c.get<uint32_t>();
    if (c.ok && version != 2 && version != 3) {  // header.rs:41
        snprintf(msg, sizeof msg, "unsupported GGUF version %u", version);
        return failf(msg);
    }
    n_tensors = c.get<uint64_t>();
    n_kv = c.get<uint64_t>();
    for (uint64_t i = 0; i < n_kv && c.ok; i++) {
        std::string key = c.str();
        const uint32_t type = c.get<uint32_t>();
        if (!c.ok) break;
        GgufValue v;
        if (!read_value(c, type, &v, 0)) {
            if (c.ok) {
                snprintf(msg, sizeof msg, "metadata key %s has unknown value type %u", key.c_str(), type);
                return failf(msg);
            }
            break;
        }
        meta[key] = std::move(v);
    }
    for (uint64_t i = 0; i < n_tensors && c.ok; i++) {
        GgufTensor t;
        t.name = c.str();
        const uint32_t nd = c.get<uint32_t>();
        if (!c.ok) break;
        if (nd > kMaxDims) {
            snprintf(msg, sizeof msg, "tensor %s has %u dimensions", t.name.c_str(), nd);
            return failf(msg);
        }
        for (uint32_t j = 0; j < nd; j++) t.shape.push_back(c.get<uint64_t>());
        t.type = c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (c.ok) tensors[t.name] = std::move(t);
    }
    if (!c.ok) {
        snprintf(msg, sizeof msg, "unexpected end of file at offset %zu", c.fail_at);
        return failf(msg);
    }
    uint32_t al = 32;
    if (get_u32("general.alignment", &al) && al != 0 && (al & (al - 1)) == 0) alignment = al;  // reader.rs:59-63
    data_offset = (c.pos + alignment - 1) & ~(size_t)(alignment - 1);
    for (auto& kv : tensors) {
        GgufTensor& t = kv.second;
        uint64_t elements = 1;
        for (uint64_t dsz : t.shape) {
            if (dsz != 0 && elements > UINT64_MAX / dsz) elements = 0;
            else elements *= dsz;
        }
        t.bytes = gguf_tensor_bytes(t.type, elements);
        if (t.bytes == 0) continue;  // a type this tier does not read: only an error if the tensor is asked for
        // data past the end of the file is reported when the tensor is asked for (reader.rs:71-76), not here
        if (data_offset > size_ || t.offset > size_ - data_offset || t.bytes > size_ - data_offset - t.offset) continue;
        t.data = base_ + data_offset + t.offset;
    }
    return true;
}

const GgufTensor* GgufFile::find(const std::string& name) const {
    auto it = tensors.find(name);
    return it == tensors.end() ? nullptr : &it->second;
}

bool GgufFile::get_u32(const std::string& key, uint32_t* out) const {
    auto it = meta.find(key);
    if (it == meta.end()) return false;
    const GgufValue& v = it->second;
    if (v.type == 4 || (v.type == 10 && v.u <= UINT32_MAX)) {
        *out = (uint32_t)v.u;
        return true;
    }
    if (v.type == 5 && v.i >= 0) {
        *out = (uint32_t)v.i;
        return true;
    }
    return false;
}

bool GgufFile::get_f32(const std::string& key, float* out) const {
    auto it = meta.find(key);
    if (it == meta.end() || (it->second.type != 6 && it->second.type != 12)) return false;
    *out = (float)it->second.f;
    return true;
}

bool GgufFile::get_str(const std::string& key, std::string* out) const {
    auto it = meta.find(key);
    if (it == meta.end() || it->second.type != 8) return false;
    *out = it->second.s;
    return true;
}

}  // namespace oxb
