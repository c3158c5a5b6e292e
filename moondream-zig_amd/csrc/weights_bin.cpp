// Reader of the converted weight file "moondream.bin" -- replaces Weights.init (weights.zig:62-204): u32 magic "MOON",
// u32 version 2, then one record per tensor: {u32 name length, u32 number of dims, u32 element count}, the name, the dims
// as u64, the elements as little-endian binary16.  The file is mapped, not read: tensors are handed to the session
// constructors as pointers into the mapping and uploaded from there, so a 3.7 GB file never sits in host memory twice.
// Host code only (no device call), which is why it also runs where no GPU is present.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "moonhip.h"

struct BinTensor {
    std::string name;
    size_t ndim = 0;
    size_t dims[4] = {0, 0, 0, 0};
    size_t numel = 0;
    const moon_f16 *data = nullptr;
};

struct moon_bin {
    int fd = -1;
    void *map = nullptr;
    size_t size = 0;
    std::vector<BinTensor> tensors;
};

namespace {

constexpr uint32_t BIN_MAGIC = 0x4D4F4F4E; // weights.zig:10
constexpr uint32_t BIN_VERSION = 2;        // weights.zig:11

int bin_fail(char *err, size_t err_len, int code, const char *fmt, ...) {
    if (err && err_len) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, err_len, fmt, ap);
        va_end(ap);
    }
    return code;
}

uint32_t rd32(const unsigned char *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
uint64_t rd64(const unsigned char *p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }

// the tensor names Weights.storeTensor accepts (weights.zig:236-318); anything else is error.UnknownTensorName
const char *const KNOWN_NAMES[] = {"word_token_embedding", "t_ln_w", "t_ln_b", "t_Wqkv_w", "t_Wqkv_b", "t_out_proj_w", "t_out_proj_bias", "t_fc1_w",
                                   "t_fc1_b", "t_fc2_w", "t_fc2_b", "t_linear_w", "t_linear_b", "t_ln_out_w", "t_ln_out_b",
                                   "v_patch_embedding_linear_w", "v_patch_embedding_linear_b", "v_pos_embedding", "v_Wqkv_w", "v_Wqkv_b",
                                   "v_out_proj_w", "v_out_proj_b", "v_fc1_w", "v_fc1_b", "v_fc2_w", "v_fc2_b", "v_norm1_w", "v_norm1_b", "v_norm2_w",
                                   "v_norm2_b", "v_norm_out_w", "v_norm_out_b", "v_proj_fc1_w", "v_proj_fc1_b", "v_proj_fc2_w", "v_proj_fc2_b"};

bool known_name(const std::string &n) {
    for (const char *k : KNOWN_NAMES)
        if (n == k) return true;
    return false;
}

const BinTensor *find(const moon_bin *bin, const char *name) {
    for (const BinTensor &t : bin->tensors)
        if (t.name == name) return &t;
    return nullptr;
}

// tensor `name` must exist with exactly the shape given (Weights.init compares with calculateShapes, weights.zig:177-181)
int want(const moon_bin *bin, const char *name, std::initializer_list<size_t> shape, const moon_f16 **out, char *err, size_t err_len) {
    const BinTensor *t = find(bin, name);
    if (!t) return bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: tensor '%s' is missing", name);
    bool ok = t->ndim == shape.size();
    size_t i = 0;
    for (size_t d : shape) {
        if (ok && t->dims[i] != d) ok = false;
        i++;
    }
    if (!ok) {
        std::string got, exp;
        for (size_t k = 0; k < t->ndim; k++) got += (k ? ", " : "") + std::to_string(t->dims[k]);
        for (size_t d : shape) exp += (exp.empty() ? "" : ", ") + std::to_string(d);
        return bin_fail(err, err_len, MOON_ESHAPE, "moondream.bin: shape mismatch for tensor '%s': got [%s], expected [%s] (ShapeMismatch)", name,
                        got.c_str(), exp.c_str());
    }
    *out = t->data;
    return MOON_OK;
}

} // namespace

extern "C" int moon_bin_open(const char *path, moon_bin **out, char *err, size_t err_len) {
    if (!path || !out) return bin_fail(err, err_len, MOON_EINVAL, "moon_bin_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: cannot open '%s': %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) {
        close(fd);
        return bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: '%s' is shorter than its 8-byte header (InvalidRead)", path);
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) {
        close(fd);
        return bin_fail(err, err_len, MOON_ENOMEM, "moondream.bin: cannot map '%s': %s", path, strerror(errno));
    }
    moon_bin *bin = new moon_bin;
    bin->fd = fd;
    bin->map = map;
    bin->size = (size_t)st.st_size;
    const unsigned char *p = (const unsigned char *)map;
    auto bail = [&](int code) {
        moon_bin_close(bin);
        return code;
    };
    if (rd32(p) != BIN_MAGIC) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: bad magic 0x%08X (InvalidMagicNumber)", rd32(p)));
    if (rd32(p + 4) != BIN_VERSION)
        return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: version %u, expected %u (InvalidVersion)", rd32(p + 4), BIN_VERSION));
    size_t pos = 8;
    while (pos < bin->size) {
        if (bin->size - pos < 12) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: truncated record header at byte %zu (InvalidHeader)", pos));
        const uint32_t name_len = rd32(p + pos), ndim = rd32(p + pos + 4), numel32 = rd32(p + pos + 8);
        pos += 12;
        if (name_len > 256) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: name length %u > 256 (InvalidNameLength)", name_len));
        if (ndim > 4) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: %u dimensions > 4 (InvalidShapeLength)", ndim));
        if (bin->size - pos < name_len + size_t(8) * ndim) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: truncated record at byte %zu (InvalidRead)", pos));
        BinTensor t;
        t.name.assign((const char *)p + pos, name_len);
        pos += name_len;
        t.ndim = ndim;
        t.numel = 1;
        for (uint32_t i = 0; i < ndim; i++) {
            const uint64_t d = rd64(p + pos);
            pos += 8;
            if (d > (uint64_t(1) << 40)) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: tensor '%s': dimension too large", t.name.c_str()));
            t.dims[i] = (size_t)d;
            // four dimensions of up to 2^40 each would wrap the product: nothing larger than the file can be meant
            if (d && t.numel > bin->size / (size_t)d)
                return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: tensor '%s': %u dimensions multiply to more elements than the file has bytes (InvalidRead)",
                                     t.name.c_str(), ndim));
            t.numel *= (size_t)d;
        }
        // the record's own element count (a u32, weights.zig:58) has to agree with the dimensions, modulo its 32 bits
        if (numel32 != (uint32_t)t.numel)
            return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: tensor '%s': header says %u elements, the dimensions %zu (InvalidHeader)",
                                 t.name.c_str(), numel32, t.numel));
        if (!known_name(t.name)) return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: unknown tensor '%s' (UnknownTensorName)", t.name.c_str()));
        if ((bin->size - pos) / 2 < t.numel)
            return bail(bin_fail(err, err_len, MOON_EFORMAT, "moondream.bin: tensor '%s' needs %zu bytes, file ends after %zu (InvalidRead)", t.name.c_str(),
                                 t.numel * 2, bin->size - pos));
        t.data = (const moon_f16 *)(p + pos);
        pos += t.numel * 2;
        bin->tensors.push_back(std::move(t));
    }
    *out = bin;
    return MOON_OK;
}

extern "C" void moon_bin_close(moon_bin *bin) {
    if (!bin) return;
    if (bin->map) munmap(bin->map, bin->size);
    if (bin->fd >= 0) close(bin->fd);
    delete bin;
}

extern "C" size_t moon_bin_tensor_count(const moon_bin *bin) { return bin ? bin->tensors.size() : 0; }

extern "C" int moon_bin_tensor(const moon_bin *bin, size_t index, const char **name, size_t *ndim, size_t dims[4], const moon_f16 **data) {
    if (!bin || index >= bin->tensors.size()) return MOON_EINVAL;
    const BinTensor &t = bin->tensors[index];
    if (name) *name = t.name.c_str();
    if (ndim) *ndim = t.ndim;
    if (dims)
        for (int i = 0; i < 4; i++) dims[i] = t.dims[i];
    if (data) *data = t.data;
    return MOON_OK;
}

extern "C" int moon_bin_find(const moon_bin *bin, const char *name, size_t *ndim, size_t dims[4], const moon_f16 **data) {
    if (!bin || !name) return MOON_EINVAL;
    for (size_t i = 0; i < bin->tensors.size(); i++)
        if (bin->tensors[i].name == name) return moon_bin_tensor(bin, i, nullptr, ndim, dims, data);
    return MOON_EFORMAT;
}

// Weights of the text decoder, shapes as calculateShapes demands them (weights.zig:439-456).
extern "C" int moon_bin_text_weights(const moon_bin *bin, const moon_text_config *c, moon_text_weights *w, char *err, size_t err_len) {
    if (!bin || !c || !w) return bin_fail(err, err_len, MOON_EINVAL, "moon_bin_text_weights: null argument");
    const size_t L = c->n_layers, d = c->dim, f = c->hidden_dim, V = c->vocab, q = c->n_heads * c->head_dim * 3;
    int rc;
#define WANT(field, name, ...)                                                                  \
    if ((rc = want(bin, name, {__VA_ARGS__}, &w->field, err, err_len)) != MOON_OK) return rc
    WANT(word_token_embedding, "word_token_embedding", V, d);
    WANT(t_ln_w, "t_ln_w", L, d);
    WANT(t_ln_b, "t_ln_b", L, d);
    WANT(t_Wqkv_w, "t_Wqkv_w", L, q, d);
    WANT(t_Wqkv_b, "t_Wqkv_b", L, q);
    WANT(t_out_proj_w, "t_out_proj_w", L, d, d);
    WANT(t_out_proj_b, "t_out_proj_bias", L, d);
    WANT(t_fc1_w, "t_fc1_w", L, f, d);
    WANT(t_fc1_b, "t_fc1_b", L, f);
    WANT(t_fc2_w, "t_fc2_w", L, d, f);
    WANT(t_fc2_b, "t_fc2_b", L, d);
    WANT(t_linear_w, "t_linear_w", V, d);
    WANT(t_linear_b, "t_linear_b", V);
    WANT(t_ln_out_w, "t_ln_out_w", d);
    WANT(t_ln_out_b, "t_ln_out_b", d);
    return MOON_OK;
}

// Weights of the vision encoder blocks (weights.zig:462-474).
extern "C" int moon_bin_vision_weights(const moon_bin *bin, const moon_vision_config *c, moon_vision_weights *w, char *err, size_t err_len) {
    if (!bin || !c || !w) return bin_fail(err, err_len, MOON_EINVAL, "moon_bin_vision_weights: null argument");
    const size_t L = c->n_layers, d = c->dim, f = c->hidden_dim, q = c->n_heads * c->head_dim * 3;
    int rc;
    WANT(v_Wqkv_w, "v_Wqkv_w", L, d, q);
    WANT(v_Wqkv_b, "v_Wqkv_b", L, q);
    WANT(v_out_proj_w, "v_out_proj_w", L, d, d);
    WANT(v_out_proj_b, "v_out_proj_b", L, d);
    WANT(v_fc1_w, "v_fc1_w", L, d, f);
    WANT(v_fc1_b, "v_fc1_b", L, f);
    WANT(v_fc2_w, "v_fc2_w", L, f, d);
    WANT(v_fc2_b, "v_fc2_b", L, d);
    WANT(v_norm1_w, "v_norm1_w", L, d);
    WANT(v_norm1_b, "v_norm1_b", L, d);
    WANT(v_norm2_w, "v_norm2_w", L, d);
    WANT(v_norm2_b, "v_norm2_b", L, d);
    WANT(v_norm_out_w, "v_norm_out_w", d);
    WANT(v_norm_out_b, "v_norm_out_b", d);
    return MOON_OK;
}

// Weights of the patch embedding, the positional embedding and the projection MLP (weights.zig:456-458, 476-479).
extern "C" int moon_bin_vision_io_weights(const moon_bin *bin, const moon_vision_config *c, const moon_vision_io_config *io,
                                          moon_vision_io_weights *w, char *err, size_t err_len) {
    if (!bin || !c || !io || !w) return bin_fail(err, err_len, MOON_EINVAL, "moon_bin_vision_io_weights: null argument");
    const size_t d = c->dim, K = io->patch_dim, T = io->tokens, Hp = io->proj_hidden, O = io->out_dim;
    int rc;
    WANT(v_patch_embedding_linear_w, "v_patch_embedding_linear_w", K, d);
    WANT(v_patch_embedding_linear_b, "v_patch_embedding_linear_b", d);
    WANT(v_pos_embedding, "v_pos_embedding", 1, T, d);
    WANT(v_proj_fc1_w, "v_proj_fc1_w", 2 * d, Hp);
    WANT(v_proj_fc1_b, "v_proj_fc1_b", Hp);
    WANT(v_proj_fc2_w, "v_proj_fc2_w", Hp, O);
    WANT(v_proj_fc2_b, "v_proj_fc2_b", O);
#undef WANT
    return MOON_OK;
}
