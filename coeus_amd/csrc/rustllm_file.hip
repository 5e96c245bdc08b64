// `.rustllm` model files: the reference's only channel for parameters (TransformerModel::write_to
// / read_from, MT:930-1121, over core/serialization.rs).  Host code only.
//
//   header   136 bytes, native (little-endian) layout of the #[repr(C)] ModelHeader
//            (serialization.rs:33-56): magic "RUSTLLM\0" @0, format_version u32 = 1 @8,
//            model_version 3 x u16 @12, padding to 24, param_count @24, param_bytes @32,
//            param_offset (= 136) @40, metadata_offset @48, metadata_size @56, checksum @64,
//            reserved 8 x u64 @72.  The reference leaves the padding uninitialised; zeros here.
//   params   little-endian f32, contiguous (serialization.rs:118-190)
//   metadata u32 len + architecture, u8 has-training-config (+ u32 len + bytes), u32 count, then
//            (u32 len + key, u32 len + value) pairs (serialization.rs:225-256)
//   checksum c = rotl1(c + bits(p)) over all parameters, wrapping u64 (serialization.rs:375-385)
//
// The reference writes five keys (hidden_dim, num_layers, num_heads, vocab_size, max_seq_len;
// MT:966-971) and rebuilds everything else from defaults (MT:1098), so a file of a model with
// another intermediate_dim or use_bias cannot be read back by it.  This writer emits the same five
// keys first, in the same order, then the remaining config fields under their field names; the
// reference looks keys up by name and ignores the extra ones.
#include "common.hpp"

#include <cerrno>
#include <cinttypes>

namespace coeus {
namespace {

constexpr uint64_t kHeaderSize = 136;
const char kMagic[8] = {'R', 'U', 'S', 'T', 'L', 'L', 'M', '\0'};

struct Header {
    uint32_t format_version = 1;
    uint16_t version[3] = {1, 0, 0};
    uint64_t param_count = 0, param_bytes = 0, param_offset = kHeaderSize, metadata_offset = 0,
             metadata_size = 0, checksum = 0;
};

void put(std::vector<uint8_t> &b, const void *p, size_t n) { b.insert(b.end(), (const uint8_t *)p, (const uint8_t *)p + n); }
void put_u32(std::vector<uint8_t> &b, uint32_t v) { put(b, &v, 4); }
void put_str(std::vector<uint8_t> &b, const std::string &s) { put_u32(b, (uint32_t)s.size()); put(b, s.data(), s.size()); }

void encode_header(const Header &h, uint8_t (&out)[kHeaderSize]) {
    std::memset(out, 0, kHeaderSize);
    std::memcpy(out, kMagic, 8);
    std::memcpy(out + 8, &h.format_version, 4);
    std::memcpy(out + 12, h.version, 6);
    std::memcpy(out + 24, &h.param_count, 8);
    std::memcpy(out + 32, &h.param_bytes, 8);
    std::memcpy(out + 40, &h.param_offset, 8);
    std::memcpy(out + 48, &h.metadata_offset, 8);
    std::memcpy(out + 56, &h.metadata_size, 8);
    std::memcpy(out + 64, &h.checksum, 8);
}

int decode_header(const uint8_t (&in)[kHeaderSize], Header &h) {
    if (std::memcmp(in, kMagic, 8) != 0) return fail(COEUS_INVALID_INPUT, "Invalid magic bytes");  // serialization.rs:77-79
    std::memcpy(&h.format_version, in + 8, 4);
    if (h.format_version != 1)  // serialization.rs:81-86
        return fail(COEUS_INVALID_INPUT, "Unsupported format version: %u", h.format_version);
    std::memcpy(h.version, in + 12, 6);
    std::memcpy(&h.param_count, in + 24, 8);
    std::memcpy(&h.param_bytes, in + 32, 8);
    std::memcpy(&h.param_offset, in + 40, 8);
    std::memcpy(&h.metadata_offset, in + 48, 8);
    std::memcpy(&h.metadata_size, in + 56, 8);
    std::memcpy(&h.checksum, in + 64, 8);
    return COEUS_OK;
}

struct File {
    FILE *f = nullptr;
    ~File() { if (f) std::fclose(f); }
};

int read_header(File &file, const char *path, Header &h) {
    file.f = std::fopen(path, "rb");
    if (!file.f) return fail(COEUS_INVALID_INPUT, "Failed to open %s: %s", path, std::strerror(errno));
    uint8_t raw[kHeaderSize];
    if (std::fread(raw, 1, kHeaderSize, file.f) != kHeaderSize)
        return fail(COEUS_INVALID_INPUT, "Failed to read header: file shorter than %" PRIu64 " bytes", kHeaderSize);
    return decode_header(raw, h);
}

bool parse_u64(const std::string &s, uint64_t &v) {
    if (s.empty()) return false;
    uint64_t r = 0;
    for (char ch : s) {
        if (ch < '0' || ch > '9') return false;
        const uint64_t d = (uint64_t)(ch - '0');
        if (r > (UINT64_MAX - d) / 10) return false;  // would wrap: not a usize (str::parse fails too)
        r = r * 10 + d;
    }
    v = r;
    return true;
}

const char *kActivation[] = {"gelu", "silu_gated"};
const char *kNorm[] = {"layernorm", "rmsnorm"};
const char *kScope[] = {"sequence", "token"};
const char *kWeight[] = {"f32", "bf16", "q8_0", "q4_0"};
const char *kKv[] = {"f32", "f16", "bf16"};

template <size_t N>
void parse_enum(const std::string &v, const char *const (&names)[N], uint32_t &out) {
    for (size_t i = 0; i < N; i++)
        if (v == names[i]) out = (uint32_t)i;
}

}  // namespace

uint64_t rustllm_checksum(const float *params, uint64_t n) {
    uint64_t c = 0;
    for (uint64_t i = 0; i < n; i++) {
        uint32_t bits;
        std::memcpy(&bits, params + i, 4);
        c += bits;
        c = (c << 1) | (c >> 63);
    }
    return c;
}

int rustllm_write(const char *path, const coeus_config &cfg, const float *params, uint64_t n) {
    Header h;
    h.param_count = n;
    h.param_bytes = n * 4;
    h.checksum = rustllm_checksum(params, n);
    std::vector<uint8_t> meta;
    put_str(meta, "transformer");
    meta.push_back(0);  // no training config
    std::vector<std::pair<std::string, std::string>> kv = {
        {"hidden_dim", std::to_string(cfg.hidden_dim)},      {"num_layers", std::to_string(cfg.num_layers)},
        {"num_heads", std::to_string(cfg.num_heads)},        {"vocab_size", std::to_string(cfg.vocab_size)},
        {"max_seq_len", std::to_string(cfg.max_seq_len)},    {"intermediate_dim", std::to_string(cfg.intermediate_dim)},
        {"use_bias", cfg.use_bias ? "true" : "false"},       {"head_dim", std::to_string(cfg.head_dim)},
        {"activation", kActivation[cfg.activation & 1]},     {"norm", kNorm[cfg.norm & 1]},
        {"norm_scope", kScope[cfg.norm_scope & 1]},          {"weight_dtype", kWeight[cfg.weight_dtype & 3]},
        {"kv_dtype", kKv[cfg.kv_dtype < 3 ? cfg.kv_dtype : 0]},
    };
    char eps[64];
    std::snprintf(eps, sizeof eps, "%.9g", (double)cfg.layer_norm_eps);
    kv.push_back({"layer_norm_eps", eps});
    put_u32(meta, (uint32_t)kv.size());
    for (auto &e : kv) { put_str(meta, e.first); put_str(meta, e.second); }
    h.metadata_offset = kHeaderSize + h.param_bytes;
    h.metadata_size = meta.size();

    File file;
    file.f = std::fopen(path, "wb");
    if (!file.f) return fail(COEUS_INVALID_INPUT, "Failed to open %s: %s", path, std::strerror(errno));
    uint8_t raw[kHeaderSize];
    encode_header(h, raw);
    bool ok = std::fwrite(raw, 1, kHeaderSize, file.f) == kHeaderSize;
    const uint64_t chunk = 2u << 20;  // 8 MB of f32 per write, as the reference (serialization.rs:113)
    for (uint64_t i = 0; ok && i < n; i += chunk) {
        const uint64_t c = n - i < chunk ? n - i : chunk;
        ok = std::fwrite(params + i, 4, c, file.f) == c;  // the host is little-endian
    }
    ok = ok && std::fwrite(meta.data(), 1, meta.size(), file.f) == meta.size();
    ok = ok && std::fflush(file.f) == 0;
    if (!ok) return fail(COEUS_INVALID_INPUT, "Failed to write %s: %s", path, std::strerror(errno));
    return COEUS_OK;
}

int rustllm_read_header(const char *path, coeus_config &cfg, uint64_t &n_params) {
    File file;
    Header h;
    COEUS_TRY(read_header(file, path, h));
    if (h.param_count > UINT64_MAX / 4 || h.param_bytes != h.param_count * 4)
        return fail(COEUS_INVALID_INPUT, "Header says %" PRIu64 " parameters in %" PRIu64 " bytes", h.param_count, h.param_bytes);
    // The header is untrusted and callers size their buffers from it: what it names has to lie
    // inside the file.
    if (std::fseek(file.f, 0, SEEK_END) != 0) return fail(COEUS_INVALID_INPUT, "Failed to seek in %s", path);
    const long end = std::ftell(file.f);
    const uint64_t file_size = end < 0 ? 0 : (uint64_t)end;
    if (h.param_offset < kHeaderSize || h.param_offset > file_size || h.param_bytes > file_size - h.param_offset)
        return fail(COEUS_INVALID_INPUT, "Header names %" PRIu64 " parameter bytes at offset %" PRIu64
                    " in a file of %" PRIu64 " bytes", h.param_bytes, h.param_offset, file_size);
    if (h.metadata_offset > file_size || h.metadata_size > file_size - h.metadata_offset)
        return fail(COEUS_INVALID_INPUT, "Header names %" PRIu64 " metadata bytes at offset %" PRIu64
                    " in a file of %" PRIu64 " bytes", h.metadata_size, h.metadata_offset, file_size);
    n_params = h.param_count;
    coeus_config_default(&cfg);  // every field the file does not name keeps its default (MT:1098)
    // ModelMetadata::from_bytes on an empty block (serialization.rs:262-264)
    if (h.metadata_size == 0) return fail(COEUS_INVALID_INPUT, "Invalid metadata format");
    if (h.metadata_size > (64u << 20)) return fail(COEUS_INVALID_INPUT, "Metadata of %" PRIu64 " bytes", h.metadata_size);
    std::vector<uint8_t> meta(h.metadata_size);
    if (std::fseek(file.f, (long)h.metadata_offset, SEEK_SET) != 0 ||
        std::fread(meta.data(), 1, meta.size(), file.f) != meta.size())
        return fail(COEUS_INVALID_INPUT, "Failed to read metadata");
    size_t cur = 0;
    auto u32 = [&](uint32_t &v) {
        if (cur + 4 > meta.size()) return false;
        std::memcpy(&v, meta.data() + cur, 4);
        cur += 4;
        return true;
    };
    auto str = [&](std::string &s) {
        uint32_t len;
        if (!u32(len) || cur + len > meta.size()) return false;
        s.assign((const char *)meta.data() + cur, len);
        cur += len;
        return true;
    };
    std::string arch, tmp;
    uint32_t count = 0;
    bool ok = str(arch) && cur < meta.size();
    if (ok) {
        const uint8_t has_cfg = meta[cur++];
        if (has_cfg) ok = str(tmp);
    }
    ok = ok && u32(count);
    for (uint32_t i = 0; ok && i < count; i++) {
        std::string k, v;
        ok = str(k) && str(v);
        if (!ok) break;
        uint64_t u;
        if (k == "hidden_dim" && parse_u64(v, u)) cfg.hidden_dim = u;
        else if (k == "num_layers" && parse_u64(v, u)) cfg.num_layers = u;
        else if (k == "num_heads" && parse_u64(v, u)) cfg.num_heads = u;
        else if (k == "vocab_size" && parse_u64(v, u)) cfg.vocab_size = u;
        else if (k == "max_seq_len" && parse_u64(v, u)) cfg.max_seq_len = u;
        else if (k == "intermediate_dim" && parse_u64(v, u)) cfg.intermediate_dim = u;
        else if (k == "head_dim" && parse_u64(v, u)) cfg.head_dim = u;
        else if (k == "use_bias") cfg.use_bias = v == "true" ? 1 : (v == "false" ? 0 : cfg.use_bias);
        else if (k == "layer_norm_eps") { float f = 0.f; if (std::sscanf(v.c_str(), "%g", &f) == 1 && f > 0.f) cfg.layer_norm_eps = f; }
        else if (k == "activation") parse_enum(v, kActivation, cfg.activation);
        else if (k == "norm") parse_enum(v, kNorm, cfg.norm);
        else if (k == "norm_scope") parse_enum(v, kScope, cfg.norm_scope);
        else if (k == "weight_dtype") parse_enum(v, kWeight, cfg.weight_dtype);
        else if (k == "kv_dtype") parse_enum(v, kKv, cfg.kv_dtype);
    }
    if (!ok) return fail(COEUS_INVALID_INPUT, "Invalid metadata format");  // serialization.rs:259-330
    return COEUS_OK;
}

int rustllm_read_parameters(const char *path, float *params, uint64_t n) {
    File file;
    Header h;
    COEUS_TRY(read_header(file, path, h));
    if (h.param_count != n)
        return fail(COEUS_INVALID_INPUT, "File holds %" PRIu64 " parameters, buffer %" PRIu64, h.param_count, n);
    if (std::fseek(file.f, (long)h.param_offset, SEEK_SET) != 0)
        return fail(COEUS_INVALID_INPUT, "Failed to seek to parameters");
    const uint64_t chunk = 2u << 20;
    for (uint64_t i = 0; i < n; i += chunk) {
        const uint64_t c = n - i < chunk ? n - i : chunk;
        if (std::fread(params + i, 4, c, file.f) != c) return fail(COEUS_INVALID_INPUT, "Failed to read parameters");
    }
    if (rustllm_checksum(params, n) != h.checksum) return fail(COEUS_INVALID_INPUT, "Checksum mismatch");  // MT:1043-1048
    return COEUS_OK;
}

}  // namespace coeus
