// MKIM weight files (src/weights.rs) -> device residency.
//
// File layout (src/weights.rs:1-18): magic "MKIM0001" | u32 n_tensors | directory | data, or
// "MKIM0002" | u32 config_len | JSON config | u32 n_tensors | directory | data.  A directory
// entry is u16 name_len | name | u8 dtype | u8 n_dims | u32 dims[n_dims] | u64 offset | u64 size,
// everything little-endian, offsets from the start of the file.  An MXFP4 blob is the packed
// nibbles (R*C/2 bytes) followed by the scale bytes (R*C/32): exactly the two arrays the kernels
// read, so a blob goes to the device as it is stored and the scale pointer is blob + R*C/2.
//
// The reader maps the file read-only as BinFile::open does (src/weights.rs:471-500) and only
// trusts the directory's (offset, size); every entry is checked against the file length and
// against blob_size (src/weights.rs:40-66) before anything is dereferenced.
#include <fcntl.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "mk_common.h"

struct mk_binfile {
    const uint8_t *data = nullptr;  // whole-file read-only mapping
    size_t len = 0;
    std::string config;  // MKIM0002 JSON block; empty for MKIM0001
    bool has_config = false;
    std::vector<std::string> names;  // directory order
    std::vector<mk_bin_entry> entries;
    std::unordered_map<std::string, size_t> index;
};

struct mk_expert_set {
    void *dev = nullptr;  // one allocation: blobs (256-byte aligned) then the six pointer arrays
    size_t bytes = 0;
    size_t n = 0;
    mk_expert_table table = {};
};

namespace {

// src/weights.rs:40-66
bool blob_size(uint8_t dtype, const mk_bin_entry &e, uint64_t *out) {
    uint64_t n = 1;
    for (int i = 0; i < e.n_dims; i++) n *= e.dims[i];
    const uint64_t r = e.n_dims >= 1 ? e.dims[0] : 0, c = e.n_dims >= 2 ? e.dims[1] : 0;
    switch (dtype) {
        case MK_DTYPE_F32:
        case MK_DTYPE_I32: *out = n * 4; return true;
        case MK_DTYPE_MXFP4: *out = r * c / 2 + r * c / 32; return e.n_dims == 2;
        case MK_DTYPE_VQ1: *out = r * c / 16; return e.n_dims == 2;
        case MK_DTYPE_MXFP4SQ: *out = r * c / 2 + r * c / 32 + 4; return e.n_dims == 2;
        default: return false;
    }
}

struct Cursor {
    const uint8_t *p;
    size_t left;
    bool take(void *dst, size_t n) {
        if (left < n) return false;
        memcpy(dst, p, n);
        p += n;
        left -= n;
        return true;
    }
};

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" void mk_bin_close(mk_binfile *f) {
    if (!f) return;
    if (f->data) munmap(const_cast<uint8_t *>(f->data), f->len);
    delete f;
}

extern "C" int mk_bin_open(const char *path, mk_binfile **out) {
    MK_REQUIRE(path && out, "null pointer");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) {
        mk_set_error("%s unreadable", path);
        return MK_ERR_INVALID;
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 12) {
        close(fd);
        mk_set_error("%s: not an MKIM file (too short)", path);
        return MK_ERR_INVALID;
    }
    void *m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (m == MAP_FAILED) {
        mk_set_error("%s: mmap failed", path);
        return MK_ERR_INVALID;
    }
    mk_binfile *f = new mk_binfile;
    f->data = (const uint8_t *)m;
    f->len = (size_t)st.st_size;
    auto fail = [&](const char *why) {
        mk_set_error("%s: %s", path, why);
        mk_bin_close(f);
        return MK_ERR_INVALID;
    };
    Cursor c{f->data, f->len};
    char magic[8];
    c.take(magic, 8);
    if (memcmp(magic, "MKIM0002", 8) == 0) {
        uint32_t clen;
        if (!c.take(&clen, 4) || c.left < clen) return fail("truncated config block");
        f->config.assign((const char *)c.p, clen);
        f->has_config = true;
        c.p += clen;
        c.left -= clen;
    } else if (memcmp(magic, "MKIM0001", 8) != 0) {
        return fail("bad magic (expected MKIM0001 or MKIM0002)");
    }
    uint32_t n;
    if (!c.take(&n, 4)) return fail("truncated directory");
    // an entry takes at least 20 bytes: a count beyond that cannot be real
    if ((uint64_t)n * 20 > c.left) return fail("tensor count exceeds the file");
    f->names.reserve(n);
    f->entries.reserve(n);
    for (uint32_t i = 0; i < n; i++) {
        uint16_t nlen;
        if (!c.take(&nlen, 2) || c.left < nlen) return fail("truncated directory");
        std::string name((const char *)c.p, nlen);
        c.p += nlen;
        c.left -= nlen;
        mk_bin_entry e = {};
        uint8_t fixed[2];
        if (!c.take(fixed, 2)) return fail("truncated directory");
        e.dtype = fixed[0];
        e.n_dims = fixed[1];
        if (e.n_dims > MK_BIN_MAX_DIMS) return fail("tensor with more than 8 dims");
        if (!c.take(e.dims, 4 * (size_t)e.n_dims) || !c.take(&e.offset, 8) || !c.take(&e.size, 8)) return fail("truncated directory");
        uint64_t want;
        if (!blob_size(e.dtype, e, &want)) return fail("unknown dtype or bad dims in the directory");
        if (want != e.size) return fail("directory size does not match dtype and dims");
        if (e.offset > f->len || e.size > f->len - e.offset) return fail("tensor data beyond the end of the file");
        f->index[name] = f->entries.size();
        f->names.push_back(std::move(name));
        f->entries.push_back(e);
    }
    *out = f;
    return MK_OK;
}

extern "C" size_t mk_bin_n_tensors(const mk_binfile *f) { return f ? f->entries.size() : 0; }

extern "C" int mk_bin_entry_at(const mk_binfile *f, size_t i, const char **name, mk_bin_entry *e) {
    MK_REQUIRE(f && i < f->entries.size(), "index out of range");
    if (name) *name = f->names[i].c_str();
    if (e) *e = f->entries[i];
    return MK_OK;
}

extern "C" int mk_bin_find(const mk_binfile *f, const char *name, mk_bin_entry *e) {
    MK_REQUIRE(f && name, "null pointer");
    auto it = f->index.find(name);
    if (it == f->index.end()) {
        mk_set_error("missing tensor: %s", name);
        return MK_ERR_INVALID;
    }
    if (e) *e = f->entries[it->second];
    return MK_OK;
}

extern "C" const void *mk_bin_blob(const mk_binfile *f, const char *name, size_t *size) {
    mk_bin_entry e;
    if (!f || !name || mk_bin_find(f, name, &e) != MK_OK) return nullptr;
    if (size) *size = (size_t)e.size;
    return f->data + e.offset;
}

extern "C" const char *mk_bin_config_json(const mk_binfile *f, size_t *len) {
    if (!f || !f->has_config) return nullptr;
    if (len) *len = f->config.size();
    return f->config.c_str();
}

extern "C" int mk_bin_mxfp4_parts(const mk_binfile *f, const char *name, const uint8_t **packed, const uint8_t **scales, size_t *rows,
                                  size_t *cols) {
    mk_bin_entry e;
    int s = mk_bin_find(f, name, &e);
    if (s != MK_OK) return s;
    if (e.dtype != MK_DTYPE_MXFP4) {
        mk_set_error("%s is not mxfp4 (dtype %d)", name, (int)e.dtype);
        return MK_ERR_INVALID;
    }
    const size_t r = e.dims[0], c = e.dims[1];
    if (packed) *packed = f->data + e.offset;
    if (scales) *scales = f->data + e.offset + r * c / 2;
    if (rows) *rows = r;
    if (cols) *cols = c;
    return MK_OK;
}

extern "C" void mk_expert_set_free(mk_expert_set *s) {
    if (!s) return;
    if (s->dev) hipFree(s->dev);
    delete s;
}

extern "C" const mk_expert_table *mk_expert_set_table(const mk_expert_set *s) { return s ? &s->table : nullptr; }
extern "C" size_t mk_expert_set_bytes(const mk_expert_set *s) { return s ? s->bytes : 0; }
extern "C" size_t mk_expert_set_count(const mk_expert_set *s) { return s ? s->n : 0; }

extern "C" int mk_bin_load_experts(const mk_binfile *f, const char *layer_prefix, size_t n_experts, mk_expert_set **out) {
    MK_REQUIRE(f && layer_prefix && out, "null pointer");
    MK_REQUIRE(n_experts >= 1 && n_experts <= 65536, "bad expert count");
    *out = nullptr;
    int rc;
    // pass 1: resolve the 3 * n blobs (the names of src/model.rs:979-989), check dtype and shapes, lay them out
    static const char *const kind[3] = {"w1", "w3", "w2"};
    struct Blob {
        const uint8_t *host;
        size_t size, half, dev_off;
    };
    std::vector<Blob> blobs(3 * n_experts);
    std::vector<char> vq(n_experts, 0);
    bool any_vq = false;
    size_t d = 0, inter = 0, off = 0;
    for (size_t e = 0; e < n_experts; e++) {
        for (int k = 0; k < 3; k++) {
            const std::string name = std::string(layer_prefix) + "block_sparse_moe.experts." + std::to_string(e) + "." + kind[k];
            mk_bin_entry en;
            if ((rc = mk_bin_find(f, name.c_str(), &en)) != MK_OK) return rc;
            if (en.dtype != MK_DTYPE_MXFP4 && en.dtype != MK_DTYPE_VQ1) {
                // MXFP4SQ experts have no device kernel (storage format only, src/mxfp4.rs:150-151)
                mk_set_error("%s has dtype %d; the device path reads mxfp4 (1) and vq1 (3)", name.c_str(), (int)en.dtype);
                return MK_ERR_UNSUPPORTED;
            }
            if (k == 0) {
                vq[e] = en.dtype == MK_DTYPE_VQ1;  // the reference takes the expert's kind from w1 (src/model.rs:988-990)
                any_vq |= vq[e];
            } else if ((en.dtype == MK_DTYPE_VQ1) != vq[e]) {
                mk_set_error("%s: dtype %d differs from the expert's w1", name.c_str(), (int)en.dtype);
                return MK_ERR_INVALID;
            }
            const size_t r = en.dims[0], c = en.dims[1];
            if (e == 0 && k == 0) {  // w1 of the first expert fixes the layer's shapes: w1, w3 [inter, d], w2 [d, inter]
                inter = r;
                d = c;
            }
            const size_t want_r = k == 2 ? d : inter, want_c = k == 2 ? inter : d;
            if (r != want_r || c != want_c) {
                mk_set_error("%s is [%zu, %zu]; expected [%zu, %zu]", name.c_str(), r, c, want_r, want_c);
                return MK_ERR_INVALID;
            }
            if (c % 32 != 0) {
                mk_set_error("%s: columns must be a multiple of 32", name.c_str());
                return MK_ERR_INVALID;
            }
            blobs[e * 3 + k] = {f->data + en.offset, (size_t)en.size, vq[e] ? 0 : r * c / 2, off};
            off = align_up(off + (size_t)en.size, 256);
        }
    }
    // one global codebook shared by every VQ1 tensor of the file (src/model.rs:995-999)
    const uint8_t *cb_host = nullptr;
    size_t cb_off = 0;
    if (any_vq) {
        mk_bin_entry en;
        if ((rc = mk_bin_find(f, "vq_codebook", &en)) != MK_OK) return rc;
        if (en.dtype != MK_DTYPE_F32 || en.size != 256 * 16 * sizeof(float)) {
            mk_set_error("vq_codebook: bad dims (want 256 x 16 f32)");
            return MK_ERR_INVALID;
        }
        cb_host = f->data + en.offset;
        cb_off = off;
        off = align_up(off + (size_t)en.size, 256);
    }
    // every expert's matrices once more in the one-launch decode kernel's order (mk_dev_moe_pack_gate_up / _down), when the
    // layer's shapes are the ones that kernel takes and MK_EXPERT_PACK is not 0: as many bytes again as the experts themselves
    const size_t pk13 = align_up(mk_moe_pack_bytes(d, inter, 0), 256), pk2 = align_up(mk_moe_pack_bytes(d, inter, 1), 256);
    const bool with_pack = !any_vq && (d == 7168 || d == 5120) && inter == 2048 && pk2 > 0 && mk_env_int("MK_EXPERT_PACK", 1) != 0;
    const size_t pack_off = off;
    if (with_pack) off += (pk13 + pk2) * n_experts;
    // and every matrix's scale bytes in K-tile order for the matrix-core kernels (mk_dev_mxfp4_scales_by_tile), when the shapes
    // allow it and MK_EXPERT_SCALE_TILES is not 0: 1/16 of the experts' bytes again
    const size_t st_per = align_up(d * inter / 32, 256);
    const bool with_st = !any_vq && d % 512 == 0 && inter % 512 == 0 && mk_env_int("MK_EXPERT_SCALE_TILES", 1) != 0;
    const size_t st_off = off;
    if (with_st) off += 3 * st_per * n_experts;
    const size_t tab_off = off, total = off + 11 * n_experts * sizeof(void *);
    mk_expert_set *s = new mk_expert_set;
    if (hipMalloc(&s->dev, total) != hipSuccess) {
        (void)hipGetLastError();
        delete s;
        mk_set_error("hipMalloc of %zu bytes for %zu experts failed", total, n_experts);
        return MK_ERR_NOMEM;
    }
    s->bytes = total;
    s->n = n_experts;
    uint8_t *base = (uint8_t *)s->dev;
    // pass 2: one copy per blob straight out of the mapping, then the pointer arrays
    std::vector<const uint8_t *> ptrs(11 * n_experts, nullptr);
    for (size_t e = 0; e < n_experts; e++) {
        for (int k = 0; k < 3; k++) {
            const Blob &b = blobs[e * 3 + k];
            if (hipMemcpy(base + b.dev_off, b.host, b.size, hipMemcpyHostToDevice) != hipSuccess) {
                (void)hipGetLastError();
                mk_expert_set_free(s);
                mk_set_error("upload of expert %zu failed", e);
                return MK_ERR_HIP;
            }
            ptrs[(size_t)(2 * k) * n_experts + e] = base + b.dev_off;                                  // packed nibbles, or VQ1 index bytes
            ptrs[(size_t)(2 * k + 1) * n_experts + e] = vq[e] ? nullptr : base + b.dev_off + b.half;  // scales (none: VQ1)
        }
    }
    for (size_t e = 0; with_pack && e < n_experts; e++) {
        uint8_t *t13 = base + pack_off + e * (pk13 + pk2), *t2 = t13 + pk13;
        if (mk_dev_moe_pack_gate_up(ptrs[e], ptrs[n_experts + e], ptrs[2 * n_experts + e], ptrs[3 * n_experts + e], d, inter, t13, nullptr) != MK_OK ||
            mk_dev_moe_pack_down(ptrs[4 * n_experts + e], ptrs[5 * n_experts + e], d, inter, t2, nullptr) != MK_OK) {
            mk_expert_set_free(s);
            return MK_ERR_HIP;
        }
        ptrs[6 * n_experts + e] = t13;
        ptrs[7 * n_experts + e] = t2;
    }
    for (size_t e = 0; with_st && e < n_experts; e++) {
        for (int k = 0; k < 3; k++) {
            uint8_t *t = base + st_off + (3 * e + k) * st_per;
            if (mk_dev_mxfp4_scales_by_tile(ptrs[(size_t)(2 * k + 1) * n_experts + e], k == 2 ? d : inter, k == 2 ? inter : d, t, nullptr) != MK_OK) {
                mk_expert_set_free(s);
                return MK_ERR_HIP;
            }
            ptrs[(size_t)(8 + k) * n_experts + e] = t;
        }
    }
    if ((with_pack || with_st) && hipDeviceSynchronize() != hipSuccess) {
        (void)hipGetLastError();
        mk_expert_set_free(s);
        mk_set_error("the packed copies of the experts failed");
        return MK_ERR_HIP;
    }
    if (cb_host && hipMemcpy(base + cb_off, cb_host, 256 * 16 * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        mk_expert_set_free(s);
        mk_set_error("upload of the VQ codebook failed");
        return MK_ERR_HIP;
    }
    if (hipMemcpy(base + tab_off, ptrs.data(), ptrs.size() * sizeof(void *), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        mk_expert_set_free(s);
        mk_set_error("upload of the expert pointer table failed");
        return MK_ERR_HIP;
    }
    const uint8_t *const *tab = (const uint8_t *const *)(base + tab_off);
    s->table.w1p = tab;
    s->table.w1s = tab + n_experts;
    s->table.w3p = tab + 2 * n_experts;
    s->table.w3s = tab + 3 * n_experts;
    s->table.w2p = tab + 4 * n_experts;
    s->table.w2s = tab + 5 * n_experts;
    s->table.d = d;
    s->table.inter = inter;
    s->table.n_experts = n_experts;
    s->table.vq_codebook = any_vq ? reinterpret_cast<const float *>(base + cb_off) : nullptr;
    s->table.w13t = with_pack ? tab + 6 * n_experts : nullptr;
    s->table.w2t = with_pack ? tab + 7 * n_experts : nullptr;
    s->table.w1st = with_st ? tab + 8 * n_experts : nullptr;
    s->table.w3st = with_st ? tab + 9 * n_experts : nullptr;
    s->table.w2st = with_st ? tab + 10 * n_experts : nullptr;
    *out = s;
    return MK_OK;
}
