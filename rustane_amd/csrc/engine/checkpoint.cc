#include "checkpoint.h"

#include "hip_decode.h"

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>

namespace rustane {
namespace {

constexpr uint32_t kVersion = 2;                  // checkpoint.rs:15
constexpr size_t kHeaderV1 = 4 + 6 * 4;           // :16
constexpr size_t kHeaderV2 = 4 + 7 * 4;           // :17

bool bad(std::string *err, const std::string &msg) {
    if (err) *err = msg;
    return false;
}

// checkpoint.rs:216-225
bool read_u32(const uint8_t *b, size_t len, size_t *cur, uint32_t *v, std::string *err) {
    if (*cur + 4 > len) return bad(err, "unexpected EOF reading u32");
    *v = (uint32_t)b[*cur] | ((uint32_t)b[*cur + 1] << 8) | ((uint32_t)b[*cur + 2] << 16) | ((uint32_t)b[*cur + 3] << 24);
    *cur += 4;
    return true;
}

// checkpoint.rs:227-247 (the host is little-endian, as every machine this backend runs on)
bool read_f32_vec(const uint8_t *b, size_t len, size_t *cur, size_t count, std::vector<float> *out, std::string *err) {
    if (count > (SIZE_MAX >> 2)) return bad(err, "checkpoint tensor size overflow");
    const size_t bytes = count * 4;
    if (bytes > len - *cur) return bad(err, "unexpected EOF reading tensor with " + std::to_string(count) + " f32 values");
    out->resize(count);
    memcpy(out->data(), b + *cur, bytes);
    *cur += bytes;
    return true;
}

// checkpoint.rs:168-214
bool infer_hidden(size_t dim, size_t nlayers, size_t vocab, size_t payload_floats, size_t *hidden, std::string *err) {
    size_t fixed, layer_fixed, denom;
    if (__builtin_mul_overflow(vocab, dim, &fixed) || __builtin_add_overflow(fixed, dim, &fixed))
        return bad(err, "checkpoint dimensions overflow");
    if (__builtin_mul_overflow((size_t)4, dim, &layer_fixed) || __builtin_mul_overflow(layer_fixed, dim, &layer_fixed) ||
        __builtin_add_overflow(layer_fixed, 2 * dim, &layer_fixed))
        return bad(err, "checkpoint dimensions overflow");
    size_t all_layers;
    if (__builtin_mul_overflow(nlayers, layer_fixed, &all_layers) || __builtin_add_overflow(all_layers, fixed, &all_layers))
        return bad(err, "checkpoint dimensions overflow");
    if (payload_floats < all_layers) return bad(err, "checkpoint payload too small for fixed-size tensors");
    const size_t hidden_total = payload_floats - all_layers;
    if (__builtin_mul_overflow(nlayers, (size_t)3, &denom) || __builtin_mul_overflow(denom, dim, &denom))
        return bad(err, "checkpoint dimensions overflow");
    if (denom == 0 || hidden_total % denom != 0)
        return bad(err, "checkpoint payload does not imply an integer hidden size");
    *hidden = hidden_total / denom;
    if (*hidden == 0) return bad(err, "checkpoint hidden size inferred as zero");
    return true;
}

}  // namespace

bool parse_checkpoint_shape(const std::string &text, CheckpointShape *out, std::string *err) {
    unsigned long long h = 0, k = 0, e = 0, f = 0;
    char tail = 0;
    const int n = sscanf(text.c_str(), " heads=%llu kv_heads=%llu hd=%llu hidden=%llu %c", &h, &k, &e, &f, &tail);
    if (n != 4) return bad(err, "checkpoint shape file must read: heads=H kv_heads=K hd=E hidden=F");
    if (!h || !k || !e || !f || h % k != 0 || e % 2 != 0)
        return bad(err, "checkpoint shape file describes no valid model (heads a multiple of kv_heads, even hd, no zeros)");
    out->heads = h; out->kv_heads = k; out->hd = e; out->hidden = f;
    return true;
}

bool parse_checkpoint(const uint8_t *bytes, size_t len, Checkpoint *out, std::string *err, const CheckpointShape *shape) {
    if (len < kHeaderV1) return bad(err, "checkpoint too small for header");
    if (memcmp(bytes, "RSTK", 4) != 0) return bad(err, "invalid checkpoint magic");
    size_t cur = 4;
    uint32_t version, step, dim, nlayers, vocab, seq, code = 0;
    if (!read_u32(bytes, len, &cur, &version, err)) return false;
    if (version < 1 || version > kVersion) return bad(err, "unsupported checkpoint version " + std::to_string(version));
    if (version >= 2 && len < kHeaderV2) return bad(err, "checkpoint too small for v2 header");
    if (!read_u32(bytes, len, &cur, &step, err) || !read_u32(bytes, len, &cur, &dim, err) ||
        !read_u32(bytes, len, &cur, &nlayers, err) || !read_u32(bytes, len, &cur, &vocab, err) ||
        !read_u32(bytes, len, &cur, &seq, err))
        return false;
    FfnActivation act = FfnActivation::SwiGlu;             // version 1 has no activation field
    if (version >= 2) {
        if (!read_u32(bytes, len, &cur, &code, err)) return false;
        if (code > 1) return bad(err, "unsupported checkpoint activation code " + std::to_string(code));   // model.rs:17-23
        act = (FfnActivation)code;
    }
    if (dim == 0 || nlayers == 0 || vocab == 0 || seq == 0) return bad(err, "checkpoint config contains zero dimension");
    if (!shape && dim % 128 != 0) return bad(err, "checkpoint dim " + std::to_string(dim) + " is not divisible by 128");
    if ((len - cur) % 4 != 0) return bad(err, "checkpoint payload is not aligned to f32 values");
    const size_t payload_floats = (len - cur) / 4;
    if (shape) {
        // The side file's numbers are not the header's: bound them as the device configuration does (32-bit
        // fields, head size 64 or 128, whole groups of query heads per key/value head) and size the payload
        // without wrap-around, so that a damaged side file cannot agree with the payload modulo 2^64.
        const uint64_t lim = 0xffffffffull;
        if (shape->heads == 0 || shape->kv_heads == 0 || shape->hidden == 0 || shape->heads > lim || shape->kv_heads > lim ||
            shape->hidden > lim || (shape->hd != 64 && shape->hd != 128) || shape->heads % shape->kv_heads != 0 ||
            shape->heads * shape->hd > lim)
            return bad(err, "checkpoint shape file holds values no model has (heads, kv_heads, hidden within 32 bits; hd 64 or 128; heads a multiple of kv_heads)");
        out->cfg = ModelConfig::make(dim, shape->hidden, shape->heads, shape->kv_heads, shape->hd, seq, nlayers, vocab, act);
        const ModelConfig &sc = out->cfg;
        size_t per_layer = 0, t = 0, total = 0;
        bool over = false;
        auto add_prod = [&](size_t a, size_t b, size_t times) {
            over |= __builtin_mul_overflow(a, b, &t) || __builtin_mul_overflow(t, times, &t) || __builtin_add_overflow(per_layer, t, &per_layer);
        };
        add_prod(sc.dim, sc.q_dim, 2);            // wq, wo
        add_prod(sc.dim, sc.kv_dim, 2);           // wk, wv
        add_prod(sc.dim, sc.hidden, 3);           // w1, w3, w2
        add_prod(sc.dim, 2, 1);                   // the two norm gains
        over |= __builtin_mul_overflow(per_layer, (size_t)sc.nlayers, &total);
        over |= __builtin_mul_overflow((size_t)sc.vocab, (size_t)sc.dim, &t) || __builtin_add_overflow(total, t, &total) ||
                __builtin_add_overflow(total, (size_t)sc.dim, &total);
        if (over || payload_floats != total)
            return bad(err, "checkpoint payload does not match the shape file beside it");
    } else {
        const size_t heads = dim / 128;
        size_t hidden = 0;
        if (!infer_hidden(dim, nlayers, vocab, payload_floats, &hidden, err)) return false;
        out->cfg = ModelConfig::make(dim, hidden, heads, heads, 128, seq, nlayers, vocab, act);
    }
    out->step = step;
    const ModelConfig &c = out->cfg;
    ModelWeights &w = out->weights;
    if (!read_f32_vec(bytes, len, &cur, c.vocab * c.dim, &w.embed, err)) return false;
    if (!read_f32_vec(bytes, len, &cur, c.dim, &w.gamma_final, err)) return false;
    w.layers.assign(c.nlayers, LayerWeights());
    for (LayerWeights &L : w.layers) {
        if (!read_f32_vec(bytes, len, &cur, c.dim * c.q_dim, &L.wq, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim * c.kv_dim, &L.wk, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim * c.kv_dim, &L.wv, err) ||
            !read_f32_vec(bytes, len, &cur, c.q_dim * c.dim, &L.wo, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim * c.hidden, &L.w1, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim * c.hidden, &L.w3, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim * c.hidden, &L.w2, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim, &L.gamma1, err) ||
            !read_f32_vec(bytes, len, &cur, c.dim, &L.gamma2, err))
            return false;
    }
    if (cur != len) return bad(err, "checkpoint had trailing bytes");
    return true;
}

bool load_checkpoint(const std::string &path, Checkpoint *out, std::string *err) {
    CheckpointShape shape;
    bool have_shape = false;
    if (FILE *sf = fopen((path + ".shape").c_str(), "r")) {
        char line[256] = {0};
        const size_t got = fread(line, 1, sizeof line - 1, sf);
        fclose(sf);
        if (!parse_checkpoint_shape(std::string(line, got), &shape, err)) return false;
        have_shape = true;
    }
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) return bad(err, "cannot open " + path + ": " + strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) { close(fd); return bad(err, "cannot stat " + path + ": " + strerror(errno)); }
    const size_t len = (size_t)st.st_size;
    if (len == 0) { close(fd); return bad(err, "checkpoint too small for header"); }
    void *p = mmap(nullptr, len, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (p == MAP_FAILED) return bad(err, "cannot map " + path + ": " + strerror(errno));
    const bool packed = len >= 4 && memcmp(p, "RSTQ", 4) == 0;
    bool ok = packed ? parse_packed_checkpoint((const uint8_t *)p, len, out, err)
                     : parse_checkpoint((const uint8_t *)p, len, out, err, have_shape ? &shape : nullptr);
    if (!ok && !packed && have_shape) {
        // A side file that does not fit the payload may be left over from an earlier file of the same name:
        // a checkpoint the header alone describes (what the reference writes) is read as such.
        std::string err2;
        Checkpoint plain;
        if (parse_checkpoint((const uint8_t *)p, len, &plain, &err2, nullptr)) {
            *out = std::move(plain);
            if (err) err->clear();
            ok = true;
        }
    }
    munmap(p, len);
    return ok;
}

namespace {
constexpr uint32_t kPackedVersion = 1;
constexpr size_t kPackedHeader = 4 + 12 * 4;
hipdec_config to_hipdec_config(const ModelConfig &c) {
    hipdec_config h{};
    h.dim = (uint32_t)c.dim; h.hidden = (uint32_t)c.hidden; h.heads = (uint32_t)c.heads; h.kv_heads = (uint32_t)c.kv_heads;
    h.hd = (uint32_t)c.hd; h.seq = (uint32_t)c.seq; h.nlayers = (uint32_t)c.nlayers; h.vocab = (uint32_t)c.vocab;
    h.q_dim = (uint32_t)c.q_dim; h.kv_dim = (uint32_t)c.kv_dim; h.gqa_ratio = (uint32_t)c.gqa_ratio;
    return h;
}
}  // namespace

bool parse_packed_checkpoint(const uint8_t *bytes, size_t len, Checkpoint *out, std::string *err) {
    if (len < kPackedHeader) return bad(err, "converted checkpoint too small for header");
    if (memcmp(bytes, "RSTQ", 4) != 0) return bad(err, "bad converted checkpoint magic");
    uint32_t h[12];
    memcpy(h, bytes + 4, sizeof h);
    if (h[0] != kPackedVersion) return bad(err, "unsupported converted checkpoint version " + std::to_string(h[0]));
    if (h[2] > 3) return bad(err, "unknown weight format " + std::to_string(h[2]) + " in converted checkpoint");
    if (h[3] > 1) return bad(err, "unknown ffn activation " + std::to_string(h[3]) + " in converted checkpoint");
    const uint32_t dim = h[4], hidden = h[5], heads = h[6], kv_heads = h[7], hd = h[8], seq = h[9], nlayers = h[10], vocab = h[11];
    if (!dim || !hidden || !heads || !kv_heads || !hd || !seq || !nlayers || !vocab || heads % kv_heads != 0)
        return bad(err, "converted checkpoint header describes no model");
    out->cfg = ModelConfig::make(dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab, (FfnActivation)h[3]);
    out->step = h[1];
    const hipdec_config hc = to_hipdec_config(out->cfg);
    hipdec_packed_sizes z;
    if (hipdec_packed_sizes_of(&hc, h[2], &z) != HIPDEC_OK)
        return bad(err, std::string("converted checkpoint: ") + hipdec_last_error(nullptr));
    const uint64_t per_layer = z.wqkv + z.s_qkv + z.wo + z.s_wo + z.w13 + z.s_w13 + z.w2 + z.s_w2 + 2 * z.gamma;
    const uint64_t want = kPackedHeader + z.gamma + z.embed + (uint64_t)nlayers * per_layer;
    if ((uint64_t)len != want)
        return bad(err, "converted checkpoint size " + std::to_string(len) + " does not match its header (" + std::to_string(want) + ")");
    auto pw = std::make_shared<PackedWeights>();
    pw->dtype = (WeightDtype)h[2];
    size_t cur = kPackedHeader;
    auto take = [&](std::vector<uint8_t> *v, uint64_t n) { v->assign(bytes + cur, bytes + cur + n); cur += n; };
    auto take_f = [&](std::vector<float> *v, uint64_t n) { v->resize(n / 4); memcpy(v->data(), bytes + cur, n); cur += n; };
    take_f(&pw->gamma_final, z.gamma);
    take(&pw->embed, z.embed);
    pw->layers.resize(nlayers);
    for (PackedLayer &L : pw->layers) {
        take(&L.wqkv, z.wqkv); take(&L.s_qkv, z.s_qkv); take(&L.wo, z.wo); take(&L.s_wo, z.s_wo);
        take(&L.w13, z.w13); take(&L.s_w13, z.s_w13); take(&L.w2, z.w2); take(&L.s_w2, z.s_w2);
        take_f(&L.gamma1, z.gamma); take_f(&L.gamma2, z.gamma);
    }
    out->weights = ModelWeights();
    out->weights.packed = pw;
    return true;
}

bool write_packed_checkpoint(const std::string &path, const ModelConfig &c, const PackedWeights &w, uint32_t step,
                             std::string *err) {
    const hipdec_config hc = to_hipdec_config(c);
    hipdec_packed_sizes z;
    if (hipdec_packed_sizes_of(&hc, (uint32_t)w.dtype, &z) != HIPDEC_OK)
        return bad(err, std::string("converted checkpoint: ") + hipdec_last_error(nullptr));
    if (w.layers.size() != c.nlayers) return bad(err, "layer count does not match the configuration");
    FILE *f = fopen(path.c_str(), "wb");
    if (!f) return bad(err, "cannot create " + path + ": " + strerror(errno));
    const uint32_t head[12] = {kPackedVersion, step, (uint32_t)w.dtype, (uint32_t)c.ffn_activation, (uint32_t)c.dim,
                               (uint32_t)c.hidden, (uint32_t)c.heads, (uint32_t)c.kv_heads, (uint32_t)c.hd, (uint32_t)c.seq,
                               (uint32_t)c.nlayers, (uint32_t)c.vocab};
    bool ok = fwrite("RSTQ", 1, 4, f) == 4 && fwrite(head, 4, 12, f) == 12;
    auto put = [&](const void *p, size_t have, uint64_t want) {
        ok = ok && have == want && (want == 0 || fwrite(p, 1, want, f) == want);
    };
    put(w.gamma_final.data(), w.gamma_final.size() * 4, z.gamma);
    put(w.embed.data(), w.embed.size(), z.embed);
    for (const PackedLayer &L : w.layers) {
        put(L.wqkv.data(), L.wqkv.size(), z.wqkv); put(L.s_qkv.data(), L.s_qkv.size(), z.s_qkv);
        put(L.wo.data(), L.wo.size(), z.wo); put(L.s_wo.data(), L.s_wo.size(), z.s_wo);
        put(L.w13.data(), L.w13.size(), z.w13); put(L.s_w13.data(), L.s_w13.size(), z.s_w13);
        put(L.w2.data(), L.w2.size(), z.w2); put(L.s_w2.data(), L.s_w2.size(), z.s_w2);
        put(L.gamma1.data(), L.gamma1.size() * 4, z.gamma); put(L.gamma2.data(), L.gamma2.size() * 4, z.gamma);
    }
    ok = (fclose(f) == 0) && ok;
    if (!ok) return bad(err, "short write or array size mismatch writing " + path);
    return true;
}

bool write_checkpoint(const std::string &path, const ModelConfig &c, const ModelWeights &w, uint32_t step,
                      std::string *err) {
    const bool needs_shape = c.hd != 128 || c.kv_heads != c.heads || c.dim != c.heads * 128;
    if (w.layers.size() != c.nlayers) return bad(err, "layer count does not match the configuration");
    const std::string shape_path = path + ".shape";
    if (needs_shape) {
        FILE *sf = fopen(shape_path.c_str(), "w");
        if (!sf) return bad(err, "cannot create " + shape_path + ": " + strerror(errno));
        const bool sok = fprintf(sf, "heads=%zu kv_heads=%zu hd=%zu hidden=%zu\n", c.heads, c.kv_heads, c.hd, c.hidden) > 0;
        if (fclose(sf) != 0 || !sok) return bad(err, "short write writing " + shape_path);
    } else {
        (void)remove(shape_path.c_str());                   // a stale side file would override the header's shape
    }
    FILE *f = fopen(path.c_str(), "wb");
    if (!f) return bad(err, "cannot create " + path + ": " + strerror(errno));
    const uint32_t head[7] = {kVersion, step, (uint32_t)c.dim, (uint32_t)c.nlayers, (uint32_t)c.vocab, (uint32_t)c.seq,
                              (uint32_t)c.ffn_activation};
    bool ok = fwrite("RSTK", 1, 4, f) == 4 && fwrite(head, 4, 7, f) == 7;
    auto put = [&](const std::vector<float> &v, size_t want) {
        ok = ok && v.size() == want && fwrite(v.data(), 4, v.size(), f) == v.size();
    };
    put(w.embed, c.vocab * c.dim);
    put(w.gamma_final, c.dim);
    for (const LayerWeights &L : w.layers) {
        put(L.wq, c.dim * c.q_dim); put(L.wk, c.dim * c.kv_dim); put(L.wv, c.dim * c.kv_dim); put(L.wo, c.q_dim * c.dim);
        put(L.w1, c.dim * c.hidden); put(L.w3, c.dim * c.hidden); put(L.w2, c.dim * c.hidden);
        put(L.gamma1, c.dim); put(L.gamma2, c.dim);
    }
    ok = (fclose(f) == 0) && ok;
    if (!ok) return bad(err, "short write or tensor size mismatch writing " + path);
    return true;
}

}  // namespace rustane
