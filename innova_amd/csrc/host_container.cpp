// host_container.cpp -- the .oil container: header, format table, tensor table, block records.
// Counterparts: OILReader (src/oil_format.cpp:289-527, include/oil/oil_format.h:66-108) and
// OILWriter (src/oil_format.cpp:189-283).  File order: 16-byte header, config bytes,
// u32 n + n x {block_id u32, format u8, cb_bytes u32}, u32 T + T x {u16 len, name, u32 start,
// u32 count}, then records [nw u32][cb_bytes u32][cb][idx_bytes u32][idx].  A tensor goes to the
// device in one pass: its records are contiguous in the file, so the mapped bytes are handed to
// oilhip_weights_create_from_records as they lie.
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "../../include/oilhip.h"

namespace oilhip {
int fail(int code, const std::string& msg);
template <typename... A>
int failf(int code, const char* fmt, A... a) {
    char b[512];
    std::snprintf(b, sizeof b, fmt, a...);
    return fail(code, b);
}
}

struct oilhip_file {
    const uint8_t* data = nullptr;
    size_t size = 0;
    bool mapped = false;
    std::vector<uint8_t> owned;
    uint32_t version = 0, flags = 0, config_size = 0;
    struct Entry { uint8_t fmt; uint32_t cb_bytes; uint32_t block_id; };
    std::vector<Entry> formats;                 // the format table, by position
    struct Tensor { std::string name; uint32_t start, count; };
    std::vector<Tensor> tensors;
    std::vector<size_t> offsets;                // record offset per block; offsets[n] = end of the last record
    size_t indexed = 0;                         // blocks whose record lies fully inside the file
    ~oilhip_file() { if (mapped && data) munmap(const_cast<uint8_t*>(data), size); }
};

namespace {

uint32_t rd32(const uint8_t* p) { uint32_t v; std::memcpy(&v, p, 4); return v; }

int parse(oilhip_file& f) {
    const uint8_t* d = f.data;
    const size_t n = f.size;
    if (n < 16) return oilhip::fail(OILHIP_E_ARG, "oil file: shorter than its 16-byte header");
    if (std::memcmp(d, "OIL1", 4) != 0) return oilhip::fail(OILHIP_E_ARG, "oil file: bad magic");
    f.version = rd32(d + 4);
    f.flags = rd32(d + 8);
    f.config_size = rd32(d + 12);
    size_t off = 16 + (size_t)f.config_size;
    if (off + 4 > n) return oilhip::fail(OILHIP_E_ARG, "oil file: truncated before the format table");
    const uint32_t nfmt = rd32(d + off);
    off += 4;
    if (off + (size_t)nfmt * 9 + 4 > n) return oilhip::fail(OILHIP_E_ARG, "oil file: truncated format table");
    f.formats.resize(nfmt);
    for (uint32_t i = 0; i < nfmt; ++i, off += 9) f.formats[i] = {d[off + 4], rd32(d + off + 5), rd32(d + off)};
    uint32_t nt = rd32(d + off);
    off += 4;
    for (uint32_t i = 0; i < nt; ++i) {          // a truncated table keeps the entries that fit (:319-326)
        if (off + 2 > n) break;
        uint16_t len;
        std::memcpy(&len, d + off, 2);
        if (off + 2 + len + 8 > n) break;
        f.tensors.push_back({std::string((const char*)d + off + 2, len), rd32(d + off + 2 + len), rd32(d + off + 6 + len)});
        off += 2 + (size_t)len + 8;
    }
    f.offsets.assign((size_t)nfmt + 1, 0);
    f.indexed = 0;
    for (uint32_t i = 0; i < nfmt; ++i) {
        f.offsets[i] = off;
        if (off + 8 > n) break;
        const uint32_t cb = rd32(d + off + 4);
        if (off + 8 + (size_t)cb + 4 > n) break;
        const uint32_t idx = rd32(d + off + 8 + cb);
        const size_t next = off + 12 + (size_t)cb + idx;
        if (next > n) break;
        off = next;
        f.indexed = i + 1;
        f.offsets[i + 1] = off;
    }
    return OILHIP_OK;
}

}  // namespace

extern "C" {

int oilhip_file_open(const char* path, oilhip_file** out) {
    if (!path || !out) return oilhip::fail(OILHIP_E_ARG, "file_open: null argument");
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) return oilhip::failf(OILHIP_E_ARG, "file_open: cannot open %s", path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) { ::close(fd); return oilhip::failf(OILHIP_E_ARG, "file_open: %s is empty or unreadable", path); }
    void* m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (m == MAP_FAILED) return oilhip::failf(OILHIP_E_NOMEM, "file_open: mmap of %s failed", path);
    auto* f = new oilhip_file;
    f->data = (const uint8_t*)m;
    f->size = (size_t)st.st_size;
    f->mapped = true;
    if (int rc = parse(*f)) { delete f; return rc; }
    *out = f;
    return OILHIP_OK;
}

int oilhip_file_open_memory(const uint8_t* bytes, uint64_t n, oilhip_file** out) {
    if (!bytes || !out) return oilhip::fail(OILHIP_E_ARG, "file_open_memory: null argument");
    *out = nullptr;
    auto* f = new oilhip_file;
    f->owned.assign(bytes, bytes + n);
    f->data = f->owned.data();
    f->size = (size_t)n;
    if (int rc = parse(*f)) { delete f; return rc; }
    *out = f;
    return OILHIP_OK;
}

int oilhip_file_close(oilhip_file* f) {
    delete f;
    return OILHIP_OK;
}

int oilhip_file_info(const oilhip_file* f, uint32_t* version, uint32_t* flags, uint32_t* config_size,
                     uint32_t* num_blocks, uint32_t* num_tensors) {
    if (!f) return oilhip::fail(OILHIP_E_ARG, "file_info: null file");
    if (version) *version = f->version;
    if (flags) *flags = f->flags;
    if (config_size) *config_size = f->config_size;
    if (num_blocks) *num_blocks = (uint32_t)f->formats.size();
    if (num_tensors) *num_tensors = (uint32_t)f->tensors.size();
    return OILHIP_OK;
}

int oilhip_file_config(const oilhip_file* f, uint8_t* out, uint32_t cap) {
    if (!f || (!out && cap)) return oilhip::fail(OILHIP_E_ARG, "file_config: null argument");
    if (cap < f->config_size) return oilhip::fail(OILHIP_E_ARG, "file_config: buffer too small");
    if (f->config_size) std::memcpy(out, f->data + 16, f->config_size);
    return OILHIP_OK;
}

int oilhip_file_tensor(const oilhip_file* f, uint32_t i, char* name, size_t name_cap, uint32_t* start,
                       uint32_t* count, uint64_t* num_weights) {
    if (!f || i >= f->tensors.size()) return oilhip::fail(OILHIP_E_ARG, "file_tensor: index out of range");
    const auto& t = f->tensors[i];
    if (name && name_cap) std::snprintf(name, name_cap, "%s", t.name.c_str());
    if (start) *start = t.start;
    if (count) *count = t.count;
    if (num_weights) {
        uint64_t total = 0;
        for (uint32_t b = 0; b < t.count; ++b)
            if ((size_t)t.start + b < f->indexed) total += rd32(f->data + f->offsets[(size_t)t.start + b]);
        *num_weights = total;
    }
    return OILHIP_OK;
}

int oilhip_file_find_tensor(const oilhip_file* f, const char* name, uint32_t* index) {
    if (!f || !name) return oilhip::fail(OILHIP_E_ARG, "file_find_tensor: null argument");
    for (size_t i = 0; i < f->tensors.size(); ++i)
        if (f->tensors[i].name == name) { if (index) *index = (uint32_t)i; return OILHIP_OK; }   // first match, like :428-433
    return oilhip::failf(OILHIP_E_ARG, "file_find_tensor: no tensor named %s", name);
}

int oilhip_file_block(const oilhip_file* f, uint32_t id, uint8_t* fmt, uint32_t* nw, const uint8_t** cb,
                      uint32_t* cb_bytes, const uint8_t** idx, uint32_t* idx_bytes) {
    if (!f || id >= f->indexed) return oilhip::failf(OILHIP_E_ARG, "file_block: block %u is not in the file", id);
    const uint8_t* p = f->data + f->offsets[id];
    const uint32_t c = rd32(p + 4), x = rd32(p + 8 + c);
    if (fmt) *fmt = f->formats[id].fmt <= 14 ? f->formats[id].fmt : (uint8_t)OILHIP_OIL32;   // :405-408
    if (nw) *nw = rd32(p);
    if (cb) *cb = p + 8;
    if (cb_bytes) *cb_bytes = c;
    if (idx) *idx = p + 12 + c;
    if (idx_bytes) *idx_bytes = x;
    return OILHIP_OK;
}

int oilhip_file_upload_tensor(const oilhip_file* f, uint32_t tensor, uint64_t rows, uint64_t cols, oilhip_weights** out) {
    if (!f || !out || tensor >= f->tensors.size()) return oilhip::fail(OILHIP_E_ARG, "file_upload_tensor: bad arguments");
    const auto& t = f->tensors[tensor];
    if (t.count == 0 || (size_t)t.start + t.count > f->indexed)
        return oilhip::failf(OILHIP_E_ARG, "file_upload_tensor: %s names blocks the file does not hold", t.name.c_str());
    std::vector<uint8_t> fmts(t.count);
    uint64_t total = 0;
    for (uint32_t b = 0; b < t.count; ++b) {
        const uint8_t wf = f->formats[(size_t)t.start + b].fmt;
        fmts[b] = wf <= 14 ? wf : (uint8_t)OILHIP_OIL32;
        total += rd32(f->data + f->offsets[(size_t)t.start + b]);
    }
    if (rows == 0 && cols == 0) { rows = 1; cols = total; }
    const size_t a = f->offsets[t.start], e = f->offsets[(size_t)t.start + t.count];
    return oilhip_weights_create_from_records(f->data + a, e - a, fmts.data(), t.count, rows, cols, out);
}

int oilhip_file_write(const char* path, uint32_t version, uint32_t flags, const uint8_t* config, uint32_t config_size,
                      uint32_t ntensors, const char* const* names, const uint32_t* tensor_blocks,
                      const uint8_t* payload, const oilhip_block_t* blocks, uint32_t nblocks) {
    if (!path || (ntensors && (!names || !tensor_blocks)) || (nblocks && (!payload || !blocks)) || (config_size && !config))
        return oilhip::fail(OILHIP_E_ARG, "file_write: null argument");
    uint64_t covered = 0;
    for (uint32_t i = 0; i < ntensors; ++i) covered += tensor_blocks[i];
    if (covered != nblocks) return oilhip::failf(OILHIP_E_ARG, "file_write: tensors cover %llu blocks, %u given", (unsigned long long)covered, nblocks);
    std::FILE* fp = std::fopen(path, "wb");
    if (!fp) return oilhip::failf(OILHIP_E_ARG, "file_write: cannot create %s", path);
    std::vector<uint8_t> buf;
    auto put = [&](const void* p, size_t n) { const uint8_t* b = (const uint8_t*)p; buf.insert(buf.end(), b, b + n); };
    auto put32 = [&](uint32_t v) { put(&v, 4); };
    put("OIL1", 4); put32(version); put32(flags); put32(config_size);
    if (config_size) put(config, config_size);
    put32(nblocks);
    for (uint32_t b = 0; b < nblocks; ++b) { put32(b); put(&blocks[b].fmt, 1); put32(blocks[b].cb_bytes); }
    put32(ntensors);
    uint32_t start = 0;
    for (uint32_t i = 0; i < ntensors; ++i) {
        const size_t len = std::strlen(names[i]);
        if (len > 0xFFFF) { std::fclose(fp); return oilhip::fail(OILHIP_E_ARG, "file_write: tensor name too long"); }
        const uint16_t l16 = (uint16_t)len;
        put(&l16, 2); put(names[i], len); put32(start); put32(tensor_blocks[i]);
        start += tensor_blocks[i];
    }
    bool ok = std::fwrite(buf.data(), 1, buf.size(), fp) == buf.size();
    buf.clear();
    for (uint32_t b = 0; b < nblocks && ok; ++b) {
        const oilhip_block_t& k = blocks[b];
        put32(k.nw); put32(k.cb_bytes); put(payload + k.cb_off, k.cb_bytes); put32(k.idx_bytes); put(payload + k.idx_off, k.idx_bytes);
        if (buf.size() > (8u << 20) || b + 1 == nblocks) { ok = std::fwrite(buf.data(), 1, buf.size(), fp) == buf.size(); buf.clear(); }
    }
    ok = (std::fclose(fp) == 0) && ok;
    return ok ? OILHIP_OK : oilhip::failf(OILHIP_E_ARG, "file_write: short write to %s", path);
}

}  // extern "C"
