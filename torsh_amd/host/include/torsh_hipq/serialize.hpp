// Persistence for the quantized path: the JSON form of QuantConfig and a binary container for
// prepared int8 weights.
//
//   export_config_to_json / import_config_from_json   crates/torsh-quantization/src/utils.rs:322-347
//       (serde_json of QuantConfig, crates/torsh-quantization/src/config.rs:94-109: unit enum
//        variants are strings, Option::None is null)
//
// The weight container has no counterpart in the reference (its ModelQuantizer discards the
// quantized weights, crates/torsh-models/src/quantization.rs:464-475).  Layout, little endian:
//   0   char[8]  magic "TQHIPQW1"
//   8   u32      kind (1 = linear [N,K], 2 = conv2d [OC,IC,KH,KW])
//   12  u32      flags (bit 0: bias present)
//   16  u64[4]   dims (linear: N, K, 0, 0; conv: OC, IC, KH, KW)
//   48  u64      offset of the int8 weights  (multiple of 256)
//   56  u64      offset of the f32 scales    (multiple of 256)
//   64  u64      offset of the f32 bias      (multiple of 256, 0 if absent)
//   72  u64      total file length
//   80  u64      FNV-1a 64 of every byte from offset 256 to the end
//   88..255      zero
// Weights are row-major with the reduction dimension contiguous, one scale per row: exactly what
// the GEMM and conv kernels read (their LDS swizzle is applied while addressing), so a loaded
// file goes to the device with one copy per section and no repacking.
#pragma once

#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <map>
#include <sstream>

#include "quantization.hpp"

namespace torsh {
namespace quantization {

namespace detail {

inline const char *name_of(DType d) {
    switch (d) {
    case DType::F32: return "F32";
    case DType::I8: return "I8";
    case DType::U8: return "U8";
    case DType::I16: return "I16";
    case DType::F16: return "F16";
    default: return "I32";
    }
}
inline const char *name_of(QScheme s) {
    static const char *n[] = {"PerTensorAffine", "PerChannelAffine", "PerTensorSymmetric", "PerChannelSymmetric",
                              "Int4PerTensor",   "Int4PerChannel",   "MixedPrecision",     "Binary",
                              "Ternary",         "GroupWise"};
    return n[static_cast<int>(s)];
}
inline const char *name_of(ObserverType o) {
    static const char *n[] = {"MinMax", "MovingAverage", "Histogram", "Percentile", "KLDivergence", "Entropy"};
    return n[static_cast<int>(o)];
}
inline const char *name_of(QuantBackend b) {
    static const char *n[] = {"Fbgemm", "Qnnpack", "Native", "Xnnpack"};
    return n[static_cast<int>(b)];
}
inline const char *name_of(ReduceRange r) { return r == ReduceRange::None ? "None" : "Reduce"; }

template <typename E>
inline bool parse_enum(const std::string &s, int count, E *out) {
    for (int i = 0; i < count; ++i)
        if (s == name_of(static_cast<E>(i))) {
            *out = static_cast<E>(i);
            return true;
        }
    return false;
}

inline std::string json_number(double v) {
    char buf[40];
    std::snprintf(buf, sizeof buf, "%.9g", v);  // 9 significant digits round-trip an f32
    return buf;
}

// A flat JSON reader for the documents this layer writes: objects of string keys whose values
// are strings, numbers, booleans, null or one nested object.  Values are returned as raw tokens.
class FlatJson {
  public:
    static Result<std::map<std::string, std::string>> parse_object(const std::string &text, size_t *pos_io = nullptr) {
        size_t pos = pos_io ? *pos_io : 0;
        std::map<std::string, std::string> out;
        auto skip = [&]() {
            while (pos < text.size() && std::isspace(static_cast<unsigned char>(text[pos]))) ++pos;
        };
        auto fail = [&](const char *what) { return TorshError::invalid_argument(std::string("JSON: ") + what); };
        skip();
        if (pos >= text.size() || text[pos] != '{') return fail("expected '{'");
        ++pos;
        skip();
        if (pos < text.size() && text[pos] == '}') {
            ++pos;
            if (pos_io) *pos_io = pos;
            return out;
        }
        for (;;) {
            skip();
            if (pos >= text.size() || text[pos] != '"') return fail("expected a string key");
            const size_t kend = text.find('"', pos + 1);
            if (kend == std::string::npos) return fail("unterminated key");
            const std::string key = text.substr(pos + 1, kend - pos - 1);
            pos = kend + 1;
            skip();
            if (pos >= text.size() || text[pos] != ':') return fail("expected ':'");
            ++pos;
            skip();
            const size_t vstart = pos;
            if (pos < text.size() && text[pos] == '{') {  // nested object: keep its text
                int depth = 0;
                do {
                    if (text[pos] == '{') ++depth;
                    if (text[pos] == '}') --depth;
                    ++pos;
                } while (pos < text.size() && depth > 0);
                if (depth != 0) return fail("unterminated object");
            } else if (pos < text.size() && text[pos] == '"') {
                const size_t vend = text.find('"', pos + 1);
                if (vend == std::string::npos) return fail("unterminated string");
                pos = vend + 1;
            } else {
                while (pos < text.size() && text[pos] != ',' && text[pos] != '}' &&
                       !std::isspace(static_cast<unsigned char>(text[pos])))
                    ++pos;
                if (pos == vstart) return fail("missing value");
            }
            out[key] = text.substr(vstart, pos - vstart);
            skip();
            if (pos < text.size() && text[pos] == ',') {
                ++pos;
                continue;
            }
            if (pos < text.size() && text[pos] == '}') {
                ++pos;
                break;
            }
            return fail("expected ',' or '}'");
        }
        if (pos_io) *pos_io = pos;
        return out;
    }
    static std::string unquote(const std::string &tok) {
        return (tok.size() >= 2 && tok.front() == '"') ? tok.substr(1, tok.size() - 2) : tok;
    }
};

}  // namespace detail

// utils.rs:322-331 (serde_json::to_string_pretty, two-space indent, field order of the struct)
inline Result<std::string> export_config_to_json(const QuantConfig &c) {
    auto opt = [](const auto &o) { return o ? std::to_string(*o) : std::string("null"); };
    std::ostringstream o;
    o << "{\n"
      << "  \"dtype\": \"" << detail::name_of(c.dtype) << "\",\n"
      << "  \"scheme\": \"" << detail::name_of(c.scheme) << "\",\n"
      << "  \"enable_fake_quant\": " << (c.enable_fake_quant ? "true" : "false") << ",\n"
      << "  \"observer_type\": \"" << detail::name_of(c.observer_type) << "\",\n"
      << "  \"backend\": \"" << detail::name_of(c.backend) << "\",\n"
      << "  \"reduce_range\": \"" << detail::name_of(c.reduce_range) << "\",\n"
      << "  \"qint_min\": " << opt(c.qint_min) << ",\n"
      << "  \"qint_max\": " << opt(c.qint_max) << ",\n"
      << "  \"eps\": " << detail::json_number(c.eps) << ",\n"
      << "  \"averaging_constant\": " << detail::json_number(c.averaging_constant) << ",\n"
      << "  \"ch_axis\": " << opt(c.ch_axis) << ",\n"
      << "  \"group_size\": " << opt(c.group_size) << "\n"
      << "}";
    return o.str();
}

// utils.rs:341-347: every field of the struct must be present, as serde requires.
inline Result<QuantConfig> import_config_from_json(const std::string &json) {
    auto parsed = detail::FlatJson::parse_object(json);
    if (parsed.is_err())
        return TorshError::invalid_argument("Failed to deserialize config: " + parsed.unwrap_err().message);
    const auto &m = parsed.unwrap();
    auto bad = [](const std::string &why) {
        return TorshError::invalid_argument("Failed to deserialize config: " + why);
    };
    for (const char *k : {"dtype", "scheme", "enable_fake_quant", "observer_type", "backend", "reduce_range",
                          "qint_min", "qint_max", "eps", "averaging_constant", "ch_axis", "group_size"})
        if (!m.count(k)) return bad(std::string("missing field `") + k + "`");
    QuantConfig c;
    const std::string dt = detail::FlatJson::unquote(m.at("dtype"));
    if (dt == "F32") c.dtype = DType::F32;
    else if (dt == "I8") c.dtype = DType::I8;
    else if (dt == "U8") c.dtype = DType::U8;
    else if (dt == "I16") c.dtype = DType::I16;
    else if (dt == "I32") c.dtype = DType::I32;
    else if (dt == "F16") c.dtype = DType::F16;
    else return bad("unknown variant `" + dt + "` for dtype");
    if (!detail::parse_enum(detail::FlatJson::unquote(m.at("scheme")), 10, &c.scheme)) return bad("unknown scheme");
    if (!detail::parse_enum(detail::FlatJson::unquote(m.at("observer_type")), 6, &c.observer_type))
        return bad("unknown observer_type");
    if (!detail::parse_enum(detail::FlatJson::unquote(m.at("backend")), 4, &c.backend)) return bad("unknown backend");
    if (!detail::parse_enum(detail::FlatJson::unquote(m.at("reduce_range")), 2, &c.reduce_range))
        return bad("unknown reduce_range");
    const std::string &fq = m.at("enable_fake_quant");
    if (fq != "true" && fq != "false") return bad("enable_fake_quant must be a boolean");
    c.enable_fake_quant = fq == "true";
    auto number = [&](const char *k, double *out) {
        char *end = nullptr;
        const std::string &t = m.at(k);
        *out = std::strtod(t.c_str(), &end);
        return end != t.c_str() && *end == '\0';
    };
    double v;
    if (!number("eps", &v)) return bad("eps must be a number");
    c.eps = static_cast<float>(v);
    if (!number("averaging_constant", &v)) return bad("averaging_constant must be a number");
    c.averaging_constant = static_cast<float>(v);
    if (m.at("qint_min") != "null") {
        if (!number("qint_min", &v)) return bad("qint_min must be an integer or null");
        c.qint_min = static_cast<int32_t>(v);
    }
    if (m.at("qint_max") != "null") {
        if (!number("qint_max", &v)) return bad("qint_max must be an integer or null");
        c.qint_max = static_cast<int32_t>(v);
    }
    if (m.at("ch_axis") != "null") {
        if (!number("ch_axis", &v) || v < 0) return bad("ch_axis must be a non-negative integer or null");
        c.ch_axis = static_cast<size_t>(v);
    }
    if (m.at("group_size") != "null") {
        if (!number("group_size", &v) || v < 0) return bad("group_size must be a non-negative integer or null");
        c.group_size = static_cast<size_t>(v);
    }
    return c;
}

// ---- prepared int8 weights on disk -------------------------------------------------------------

// Where byte (row, k) of an int8 matrix [rows, K] lives in the operand order of the matrix cores (the layout
// hipq_pack_rows_i8 writes): [row block of 32][k block of 32 bytes, padded to a multiple of 4][1 KiB], and inside a
// fragment slot l = row % 32 + 32 * ((k % 32) / 16) of 16 bytes.  Padding rows and k are zero.
namespace packed_layout {
inline size_t k_blocks(size_t k) { return ((k + 31) / 32 + 3) / 4 * 4; }
inline size_t bytes(size_t rows, size_t k) { return ((rows + 31) / 32) * k_blocks(k) * 1024; }
inline size_t offset(size_t row, size_t kk, size_t k) {
    return ((row / 32) * k_blocks(k) + kk / 32) * 1024 + ((kk % 32) / 16) * 512 + (row % 32) * 16 + kk % 16;
}
inline std::vector<int8_t> unpack(const std::vector<int8_t> &packed, size_t rows, size_t k) {
    std::vector<int8_t> out(rows * k);
    for (size_t r = 0; r < rows; ++r)
        for (size_t kk = 0; kk < k; ++kk) out[r * k + kk] = packed[offset(r, kk, k)];
    return out;
}
}  // namespace packed_layout

struct QuantizedWeights {
    enum Kind : uint32_t { Linear = 1, Conv2d = 2 };
    Kind kind = Linear;
    std::vector<size_t> dims;    // [N, K] or [OC, IC, KH, KW]
    std::vector<int8_t> weight;  // rows() x row_len(), row-major
    std::vector<float> scales;   // one per row
    std::vector<float> bias;     // empty or one per row
    // Linear only, optional: the same rows already in the operand order of the matrix cores
    // (packed_layout::bytes(N, K) bytes).  A file saved with it holds the prepared operand instead of the
    // row-major rows, and a layer loaded from such a file uploads it as it is: no packing pass on the device.
    std::vector<int8_t> packed;

    size_t rows() const { return dims.empty() ? 0 : dims[0]; }
    size_t row_len() const {
        size_t n = 1;
        for (size_t i = 1; i < dims.size(); ++i) n *= dims[i];
        return dims.size() > 1 ? n : 0;
    }
    Result<Unit> validate() const {
        if (kind == Linear && dims.size() != 2) return TorshError::invalid_argument("linear weights need dims [N, K]");
        if (kind == Conv2d && dims.size() != 4)
            return TorshError::invalid_argument("conv2d weights need dims [OC, IC, KH, KW]");
        if (kind != Linear && kind != Conv2d) return TorshError::invalid_argument("unknown weight kind");
        if (weight.size() != rows() * row_len() || scales.size() != rows() || (!bias.empty() && bias.size() != rows()))
            return TorshError::invalid_argument("quantized weight sections do not match dims");
        if (!packed.empty() && (kind != Linear || packed.size() != packed_layout::bytes(rows(), row_len())))
            return TorshError::invalid_argument("prepared weight section does not match dims");
        return Unit{};
    }
};

namespace detail {
inline uint64_t fnv1a64(const unsigned char *p, size_t n, uint64_t h = 1469598103934665603ull) {
    for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
    return h;
}
inline size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
constexpr char kWeightMagic[8] = {'T', 'Q', 'H', 'I', 'P', 'Q', 'W', '2'};
// a * b without wrapping; false when the product does not fit
inline bool mul_fits(uint64_t a, uint64_t b, uint64_t *out) { return !__builtin_mul_overflow(a, b, out); }
}  // namespace detail

inline Result<Unit> save_quantized_weights(const QuantizedWeights &w, const std::string &path) {
    TORSH_CHECK(w.validate());
    const size_t off_w = 256;
    // flag 2: the weight section is the prepared operand (tile order), not the row-major rows
    const std::vector<int8_t> &payload = w.packed.empty() ? w.weight : w.packed;
    const size_t off_s = detail::align256(off_w + payload.size());
    const size_t off_b = w.bias.empty() ? 0 : detail::align256(off_s + w.scales.size() * sizeof(float));
    const size_t total = detail::align256(w.bias.empty() ? off_s + w.scales.size() * sizeof(float)
                                                         : off_b + w.bias.size() * sizeof(float));
    std::vector<unsigned char> buf(total, 0);
    std::memcpy(buf.data(), detail::kWeightMagic, 8);
    const uint32_t kind = w.kind, flags = (w.bias.empty() ? 0u : 1u) | (w.packed.empty() ? 0u : 2u);
    std::memcpy(buf.data() + 8, &kind, 4);
    std::memcpy(buf.data() + 12, &flags, 4);
    uint64_t dims[4] = {0, 0, 0, 0};
    for (size_t i = 0; i < w.dims.size(); ++i) dims[i] = w.dims[i];
    std::memcpy(buf.data() + 16, dims, 32);
    const uint64_t offs[4] = {off_w, off_s, off_b, total};
    std::memcpy(buf.data() + 48, offs, 32);
    std::memcpy(buf.data() + off_w, payload.data(), payload.size());
    std::memcpy(buf.data() + off_s, w.scales.data(), w.scales.size() * sizeof(float));
    if (!w.bias.empty()) std::memcpy(buf.data() + off_b, w.bias.data(), w.bias.size() * sizeof(float));
    // the checksum covers the header too (its own field counted as zero), so a damaged dimension or offset is
    // caught before it is used
    const uint64_t sum = detail::fnv1a64(buf.data(), total);
    std::memcpy(buf.data() + 80, &sum, 8);
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    if (!f) return TorshError::invalid_argument("Failed to open " + path + " for writing");
    f.write(reinterpret_cast<const char *>(buf.data()), static_cast<std::streamsize>(total));
    if (!f) return TorshError::invalid_argument("Failed to write " + path);
    return Unit{};
}

inline Result<QuantizedWeights> load_quantized_weights(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return TorshError::invalid_argument("Failed to open " + path);
    std::vector<unsigned char> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    auto bad = [&](const char *why) { return TorshError::invalid_argument(path + ": " + why); };
    // (the row / length extraction below needs them before the sections are read)
    if (buf.size() < 256 || std::memcmp(buf.data(), detail::kWeightMagic, 8) != 0)
        return bad("not a quantized-weight file");
    uint32_t kind, flags;
    uint64_t dims[4], offs[4], sum;
    std::memcpy(&kind, buf.data() + 8, 4);
    std::memcpy(&flags, buf.data() + 12, 4);
    std::memcpy(dims, buf.data() + 16, 32);
    std::memcpy(offs, buf.data() + 48, 32);
    std::memcpy(&sum, buf.data() + 80, 8);
    if (offs[3] != buf.size()) return bad("length field does not match the file (truncated?)");
    {
        std::vector<unsigned char> zeroed(buf.begin(), buf.begin() + 256);
        std::memset(zeroed.data() + 80, 0, 8);
        const uint64_t h = detail::fnv1a64(buf.data() + 256, buf.size() - 256, detail::fnv1a64(zeroed.data(), 256));
        if (h != sum) return bad("checksum mismatch");
    }
    QuantizedWeights w;
    if (kind != QuantizedWeights::Linear && kind != QuantizedWeights::Conv2d) return bad("unknown weight kind");
    w.kind = static_cast<QuantizedWeights::Kind>(kind);
    const size_t nd = kind == QuantizedWeights::Linear ? 2 : 4;
    for (size_t i = 0; i < nd; ++i) w.dims.push_back(static_cast<size_t>(dims[i]));
    // every product and sum below is checked: the fields come from the file
    uint64_t len64 = 1;
    for (size_t i = 1; i < nd; ++i)
        if (!detail::mul_fits(len64, dims[i], &len64)) return bad("implausible dims");
    const uint64_t rows64 = dims[0], size = buf.size();
    uint64_t wbytes = 0, fbytes = 0;
    if (rows64 == 0 || len64 == 0 || !detail::mul_fits(rows64, len64, &wbytes) || wbytes > size ||
        !detail::mul_fits(rows64, sizeof(float), &fbytes) || fbytes > size)
        return bad("implausible dims");
    const size_t rows = static_cast<size_t>(rows64), len = static_cast<size_t>(len64);
    const bool has_bias = (flags & 1u) != 0, prepared = (flags & 2u) != 0;
    if (flags & ~3u) return bad("unknown flags");
    if (prepared && kind != QuantizedWeights::Linear) return bad("a prepared operand belongs to linear weights");
    auto inside = [&](uint64_t off, uint64_t need) { return off >= 256 && off <= size && need <= size - off; };
    const uint64_t payload_bytes = prepared ? packed_layout::bytes(rows, len) : wbytes;  // (rows * len fits: wbytes does)
    if (!inside(offs[0], payload_bytes) || !inside(offs[1], fbytes) || (has_bias && !inside(offs[2], fbytes)))
        return bad("section outside the file");
    const int8_t *payload = reinterpret_cast<const int8_t *>(buf.data() + offs[0]);
    if (prepared) {
        w.packed.assign(payload, payload + payload_bytes);
        w.weight = packed_layout::unpack(w.packed, rows, len);  // the row-major view, for parameters() and checks
    } else {
        w.weight.assign(payload, payload + rows * len);
    }
    w.scales.resize(rows);
    std::memcpy(w.scales.data(), buf.data() + offs[1], rows * sizeof(float));
    if (has_bias) {
        w.bias.resize(rows);
        std::memcpy(w.bias.data(), buf.data() + offs[2], rows * sizeof(float));
    }
    TORSH_CHECK(w.validate());
    return w;
}

}  // namespace quantization
}  // namespace torsh
