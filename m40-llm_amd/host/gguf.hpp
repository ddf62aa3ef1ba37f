// GGUF ingestion, host side: file parser, tensor views over the data section, model configuration from
// metadata, tensor-name mapping and the lm_head / tied-embedding rules.  Pure host code: nothing here touches
// the GPU (the device loader that uses it is in gguf_loader.hpp).
//
// Behaviour follows the reference's src/gguf.rs:172-329 (parser, data-section offset), src/infer/load.rs:41-63
// and src/infer/tensor_views.rs:8-117 (bounds, alignment, strides), src/infer/types.rs:114-242 with
// src/infer/meta.rs:5-154 (configuration) and src/infer/mapping.rs:95-493 (names, shapes, dtypes), including
// the text of its error messages.  The file is mapped read-only and parsed in place with bounds checks, so a
// truncated or hostile header cannot make the parser read or allocate beyond the file.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace m40host {
namespace gguf {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// Metadata value types, src/gguf.rs:14-53.
enum ValueType : uint32_t { kU8 = 0, kI8, kU16, kI16, kU32, kI32, kF32, kBool, kStr, kArray, kU64, kI64, kF64 };

struct Scalar {
    uint32_t type = kU8;
    uint64_t u = 0;   // unsigned types and bool
    int64_t i = 0;    // signed types
    double f = 0.0;   // kF32 (exactly representable) and kF64
    std::string s;
};

struct Value {
    bool is_array = false;
    uint32_t elem_type = kU8;
    Scalar scalar;
    std::vector<Scalar> array;
};

// ggml dtype codes (src/gguf.rs:110-131) with elements and bytes per block (src/gguf.rs:305-322).
struct DTypeLayout {
    uint32_t code;
    const char* name;
    uint64_t block_elems, block_bytes;
};
inline const DTypeLayout* dtype_layout(uint32_t raw) {
    static const DTypeLayout table[] = {
        {0, "F32", 1, 4},      {1, "F16", 1, 2},      {2, "Q4_0", 32, 18},   {3, "Q4_1", 32, 20},   {6, "Q5_0", 32, 22},
        {7, "Q5_1", 32, 36},   {8, "Q8_0", 32, 34},   {9, "Q8_1", 32, 36},   {10, "Q2K", 256, 84},  {11, "Q3K", 256, 110},
        {12, "Q4K", 256, 144}, {13, "Q5K", 256, 176}, {14, "Q6K", 256, 210}, {15, "Q8K", 256, 292},
    };
    for (const auto& e : table)
        if (e.code == raw) return &e;
    return nullptr;
}
inline std::string dtype_name(uint32_t raw) {
    const DTypeLayout* l = dtype_layout(raw);
    return l ? std::string(l->name) : "Unknown(" + std::to_string(raw) + ")";
}
constexpr uint32_t kF32Code = 0, kF16Code = 1, kQ51Code = 7, kQ80Code = 8;

struct TensorInfo {
    std::string name;
    uint32_t dtype = 0;
    std::vector<uint64_t> shape;
    uint64_t offset = 0;   // from the start of the data section
};

struct TensorView {   // src/infer/types.rs DeviceTensorView without the device pointer
    uint32_t dtype = 0;
    std::vector<uint64_t> shape;
    std::vector<uint64_t> strides;   // elements, contiguous in shape order
    uint64_t byte_offset = 0, nbytes = 0;
};

inline std::string shape_text(const std::vector<uint64_t>& s) {
    std::string out = "[";
    for (size_t i = 0; i < s.size(); ++i) out += (i ? ", " : "") + std::to_string(s[i]);
    return out + "]";
}

class MappedFile {
public:
    explicit MappedFile(const std::string& path) {
        fd_ = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
        if (fd_ < 0) throw Error("failed to open GGUF file \"" + path + "\": " + std::strerror(errno));
        struct stat st {};
        if (::fstat(fd_, &st) != 0 || st.st_size < 0) {
            ::close(fd_);
            throw Error("failed to stat GGUF file \"" + path + "\"");
        }
        len_ = static_cast<uint64_t>(st.st_size);
        if (len_ > 0) {
            void* p = ::mmap(nullptr, len_, PROT_READ, MAP_PRIVATE, fd_, 0);
            if (p == MAP_FAILED) {
                ::close(fd_);
                throw Error("failed to map GGUF file \"" + path + "\"");
            }
            base_ = static_cast<const uint8_t*>(p);
        }
    }
    ~MappedFile() {
        if (base_) ::munmap(const_cast<uint8_t*>(base_), len_);
        if (fd_ >= 0) ::close(fd_);
    }
    MappedFile(const MappedFile&) = delete;
    MappedFile& operator=(const MappedFile&) = delete;
    const uint8_t* data() const { return base_; }
    uint64_t size() const { return len_; }
    int fd() const { return fd_; }

private:
    int fd_ = -1;
    const uint8_t* base_ = nullptr;
    uint64_t len_ = 0;
};

class Cursor {
public:
    Cursor(const uint8_t* p, uint64_t n) : p_(p), n_(n) {}
    uint64_t pos() const { return at_; }
    const uint8_t* take(uint64_t n) {
        if (n > n_ - at_) throw Error("failed to fill whole buffer");   // what read_exact reports at end of file
        const uint8_t* out = p_ + at_;
        at_ += n;
        return out;
    }
    template <typename T>
    T le() {
        T v;
        std::memcpy(&v, take(sizeof(T)), sizeof(T));   // little-endian host
        return v;
    }
    std::string string() {   // src/gguf.rs:368-375: u64 length, raw bytes, must be UTF-8
        const uint64_t n = le<uint64_t>();
        const uint8_t* b = take(n);
        std::string s(reinterpret_cast<const char*>(b), n);
        if (!valid_utf8(s)) throw Error("GGUF string is not valid UTF-8");
        return s;
    }
    Scalar scalar(uint32_t vt) {   // src/gguf.rs:377-421
        Scalar s;
        s.type = vt;
        switch (vt) {
            case kU8: s.u = le<uint8_t>(); break;
            case kI8: s.i = le<int8_t>(); break;
            case kU16: s.u = le<uint16_t>(); break;
            case kI16: s.i = le<int16_t>(); break;
            case kU32: s.u = le<uint32_t>(); break;
            case kI32: s.i = le<int32_t>(); break;
            case kU64: s.u = le<uint64_t>(); break;
            case kI64: s.i = le<int64_t>(); break;
            case kF32: s.f = le<float>(); break;
            case kF64: s.f = le<double>(); break;
            case kBool: s.u = le<uint8_t>() != 0; break;
            case kStr: s.s = string(); break;
            default: throw Error("read_scalar called with ARRAY type");
        }
        return s;
    }

private:
    static bool valid_utf8(const std::string& s) {
        const auto* b = reinterpret_cast<const unsigned char*>(s.data());
        const size_t n = s.size();
        for (size_t i = 0; i < n;) {
            const unsigned c = b[i];
            size_t extra;
            uint32_t cp;
            if (c < 0x80) { ++i; continue; }
            if (c >= 0xc2 && c <= 0xdf) { extra = 1; cp = c & 0x1f; }
            else if (c >= 0xe0 && c <= 0xef) { extra = 2; cp = c & 0x0f; }
            else if (c >= 0xf0 && c <= 0xf4) { extra = 3; cp = c & 0x07; }
            else return false;
            if (i + extra >= n) return false;
            for (size_t k = 1; k <= extra; ++k) {
                if ((b[i + k] & 0xc0) != 0x80) return false;
                cp = (cp << 6) | (b[i + k] & 0x3f);
            }
            if (extra == 2 && (cp < 0x800 || (cp >= 0xd800 && cp <= 0xdfff))) return false;
            if (extra == 3 && (cp < 0x10000 || cp > 0x10ffff)) return false;
            i += extra + 1;
        }
        return true;
    }
    const uint8_t* p_;
    uint64_t n_, at_ = 0;
};

inline uint64_t align_offset(uint64_t offset, uint64_t alignment) {   // src/gguf.rs:293-301
    const uint64_t rem = offset % alignment;
    return rem == 0 ? offset : offset + (alignment - rem);
}

inline bool mul_overflow(uint64_t a, uint64_t b, uint64_t* out) { return __builtin_mul_overflow(a, b, out); }
inline bool add_overflow(uint64_t a, uint64_t b, uint64_t* out) { return __builtin_add_overflow(a, b, out); }

// End of a tensor's payload relative to the data section; nullopt for unknown dtypes or on overflow
// (src/gguf.rs:303-329).
inline std::optional<uint64_t> tensor_payload_end(const TensorInfo& t) {
    const DTypeLayout* l = dtype_layout(t.dtype);
    if (!l) return std::nullopt;
    uint64_t elems = 1;
    for (uint64_t d : t.shape)
        if (mul_overflow(elems, d, &elems)) return std::nullopt;
    const uint64_t blocks = elems / l->block_elems + (elems % l->block_elems != 0);
    uint64_t bytes, end;
    if (mul_overflow(blocks, l->block_bytes, &bytes) || add_overflow(t.offset, bytes, &end)) return std::nullopt;
    return end;
}

struct Model {   // src/gguf.rs GgufModel
    uint32_t version = 0;
    std::map<std::string, Value> metadata;   // a repeated key keeps its last value, as a HashMap insert does
    std::vector<TensorInfo> tensors;
    uint64_t data_offset = 0;
    uint64_t file_len = 0;
};

inline Model parse(const uint8_t* data, uint64_t len) {   // src/gguf.rs:172-289
    Cursor c(data, len);
    if (std::memcmp(c.take(4), "GGUF", 4) != 0) throw Error("Not a GGUF file (magic != GGUF)");
    Model m;
    m.file_len = len;
    m.version = c.le<uint32_t>();
    const uint64_t n_tensors = c.le<uint64_t>();
    const uint64_t n_kv = c.le<uint64_t>();
    for (uint64_t k = 0; k < n_kv; ++k) {
        std::string key = c.string();
        const uint32_t vt = c.le<uint32_t>();
        if (vt > kF64) throw Error("unknown GGUF value type: " + std::to_string(vt));
        Value v;
        if (vt == kArray) {
            v.is_array = true;
            v.elem_type = c.le<uint32_t>();
            if (v.elem_type > kF64) throw Error("unknown GGUF array element type: " + std::to_string(v.elem_type));
            const uint64_t n = c.le<uint64_t>();
            if (v.elem_type == kArray) throw Error("read_scalar called with ARRAY type");
            if (n > len) throw Error("failed to fill whole buffer");   // every element takes at least one byte
            v.array.reserve(n);
            for (uint64_t i = 0; i < n; ++i) v.array.push_back(c.scalar(v.elem_type));
        } else {
            v.scalar = c.scalar(vt);
        }
        m.metadata[std::move(key)] = std::move(v);
    }
    for (uint64_t t = 0; t < n_tensors; ++t) {
        TensorInfo info;
        info.name = c.string();
        const uint32_t nd = c.le<uint32_t>();
        if (static_cast<uint64_t>(nd) * 8 > len) throw Error("failed to fill whole buffer");
        info.shape.reserve(nd);
        for (uint32_t i = 0; i < nd; ++i) info.shape.push_back(c.le<uint64_t>());
        info.dtype = c.le<uint32_t>();
        info.offset = c.le<uint64_t>();
        m.tensors.push_back(std::move(info));
    }
    // Offsets are relative to the aligned data section.  With no general.alignment key the default of 32 is
    // applied only when the padded payload still fits in the file (files written without padding exist).
    const uint64_t info_end = c.pos();
    uint64_t max_end = 0;
    for (const auto& t : m.tensors)
        if (auto e = tensor_payload_end(t)) max_end = std::max(max_end, *e);
    const auto it = m.metadata.find("general.alignment");
    if (it != m.metadata.end()) {
        const Value& v = it->second;
        uint64_t a = 0;
        if (!v.is_array) {
            if (v.scalar.type == kU32 || v.scalar.type == kU64) a = v.scalar.u;
            else if ((v.scalar.type == kI32 || v.scalar.type == kI64) && v.scalar.i > 0) a = static_cast<uint64_t>(v.scalar.i);
        }
        if (a == 0) throw Error("general.alignment must be a positive integer when present");
        m.data_offset = align_offset(info_end, a);
    } else if (!m.tensors.empty()) {
        const uint64_t aligned = align_offset(info_end, 32);
        uint64_t sum;
        m.data_offset = (!add_overflow(aligned, max_end, &sum) && sum <= len) ? aligned : info_end;
    } else {
        m.data_offset = info_end;
    }
    return m;
}

// ---- metadata accessors, src/infer/meta.rs:5-21, 139-154 ------------------------------------------------
using Metadata = std::map<std::string, Value>;

inline std::optional<uint32_t> get_u32(const Metadata& md, const std::string& key) {
    const auto it = md.find(key);
    if (it == md.end() || it->second.is_array) return std::nullopt;
    const Scalar& s = it->second.scalar;
    if (s.type == kU32 || s.type == kU64) return s.u <= 0xffffffffull ? std::optional<uint32_t>(static_cast<uint32_t>(s.u)) : std::nullopt;
    if (s.type == kI32 || s.type == kI64)
        return (s.i >= 0 && s.i <= 0xffffffffll) ? std::optional<uint32_t>(static_cast<uint32_t>(s.i)) : std::nullopt;
    return std::nullopt;
}
inline std::optional<uint32_t> get_u32_any(const Metadata& md, std::initializer_list<std::string> keys) {
    for (const auto& k : keys)
        if (auto v = get_u32(md, k)) return v;
    return std::nullopt;
}
inline std::optional<float> get_f32_any(const Metadata& md, std::initializer_list<std::string> keys) {
    for (const auto& k : keys) {
        const auto it = md.find(k);
        if (it != md.end() && !it->second.is_array && it->second.scalar.type == kF32) return static_cast<float>(it->second.scalar.f);
    }
    return std::nullopt;
}
inline const TensorInfo* find_tensor(const std::vector<TensorInfo>& ts, const std::string& name) {
    for (const auto& t : ts)
        if (t.name == name) return &t;
    return nullptr;
}

struct Config {   // src/infer/types.rs:17-31
    std::string architecture;
    uint32_t block_count = 0, context_length = 0, embedding_length = 0, feed_forward_length = 0, attention_head_count = 0,
             attention_head_count_kv = 0, attention_key_length = 0, vocab_size = 0;
    float layer_norm_epsilon = 1e-5f, rope_freq_base = 10000.0f, rope_freq_scale = 1.0f;
    uint32_t rope_layout() const { return architecture.rfind("qwen", 0) == 0 ? 1u : 0u; }   // types.rs:34-40
};

inline const std::vector<std::string>& embedding_names() {
    static const std::vector<std::string> names = {"tok_embeddings.weight", "token_embd.weight", "token_embd",
                                                   "token_embeddings.weight"};
    return names;
}

inline Config config_from_metadata(const Metadata& md, const std::vector<TensorInfo>& tensors) {   // types.rs:114-242
    const auto ait = md.find("general.architecture");
    if (ait == md.end() || ait->second.is_array || ait->second.scalar.type != kStr) throw Error("missing general.architecture");
    Config c;
    c.architecture = ait->second.scalar.s;
    const std::string a = c.architecture + ".";
    auto need = [&](const std::string& suffix) {
        auto v = get_u32_any(md, {a + suffix, "llama." + suffix});
        if (!v) throw Error("missing architecture " + suffix);
        return *v;
    };
    c.embedding_length = need("embedding_length");
    c.attention_head_count = need("attention.head_count");
    c.block_count = need("block_count");
    c.context_length = need("context_length");
    const uint32_t d = c.embedding_length;
    // feed_forward_length: metadata, else the first FFN weight of layer 0 shaped [d_model, H] (meta.rs:99-137)
    if (auto ff = get_u32_any(md, {a + "feed_forward_length", "llama.feed_forward_length"})) {
        if (*ff == 0) throw Error("feed_forward_length must be > 0");
        c.feed_forward_length = *ff;
    } else {
        bool found = false;
        for (const char* name : {"layers.0.feed_forward.w1.weight", "layers.0.feed_forward.w3.weight", "blk.0.ffn_gate.weight",
                                 "blk.0.ffn_up.weight", "layers.0.ffn_gate.weight", "layers.0.ffn_up.weight"}) {
            const TensorInfo* t = find_tensor(tensors, name);
            if (!t) continue;
            if (t->shape.size() != 2) throw Error(std::string("feed-forward tensor ") + name + " must be rank-2");
            const uint32_t k = static_cast<uint32_t>(t->shape[0]), n = static_cast<uint32_t>(t->shape[1]);
            if (k == d && n > 0) {
                c.feed_forward_length = n;
                found = true;
                break;
            }
        }
        if (!found)
            throw Error("feed_forward_length missing; add architecture feed_forward_length or a feed-forward weight tensor");
    }
    if (auto hd = get_u32_any(md, {a + "attention.key_length", "llama.attention.key_length"})) {
        c.attention_key_length = *hd;
    } else {
        if (c.attention_head_count == 0) throw Error("attention_head_count must be > 0");
        c.attention_key_length = d / c.attention_head_count;
    }
    // kv heads: metadata, else the K (then V) projection of layer 0, else the query head count (meta.rs:23-58)
    if (auto kv = get_u32_any(md, {a + "attention.head_count_kv", "llama.attention.head_count_kv"})) {
        c.attention_head_count_kv = *kv;
    } else {
        c.attention_head_count_kv = c.attention_head_count;
        for (const char* name : {"layers.0.attention.wk.weight", "blk.0.attn_k.weight", "layers.0.attention.wv.weight",
                                 "blk.0.attn_v.weight"}) {
            const TensorInfo* t = find_tensor(tensors, name);
            if (!t) continue;
            if (t->shape.size() != 2) throw Error(std::string("attention tensor ") + name + " must be rank-2");
            const uint32_t k = static_cast<uint32_t>(t->shape[0]), n = static_cast<uint32_t>(t->shape[1]);
            if (k == d && n > 0 && c.attention_key_length > 0 && n % c.attention_key_length == 0) {
                c.attention_head_count_kv = n / c.attention_key_length;
                break;
            }
        }
    }
    c.layer_norm_epsilon =
        get_f32_any(md, {a + "attention.layer_norm_rms_epsilon", a + "layer_norm_epsilon", "llama.layer_norm_epsilon"}).value_or(1e-5f);
    c.rope_freq_base = get_f32_any(md, {a + "rope.freq_base", "llama.rope.freq_base"}).value_or(10000.0f);
    c.rope_freq_scale = get_f32_any(md, {a + "rope.freq_scale", "llama.rope.freq_scale"}).value_or(1.0f);
    // vocab: metadata, else the embedding table's other dimension (meta.rs:60-97)
    if (auto v = get_u32_any(md, {a + "vocab_size", "llama.vocab_size"})) {
        if (*v == 0) throw Error("vocab_size must be > 0");
        c.vocab_size = *v;
    } else {
        bool found = false;
        for (const auto& name : embedding_names()) {
            const TensorInfo* t = find_tensor(tensors, name);
            if (!t) continue;
            if (t->shape.size() != 2) throw Error("embedding tensor " + name + " must be rank-2");
            const uint32_t r0 = static_cast<uint32_t>(t->shape[0]), r1 = static_cast<uint32_t>(t->shape[1]);
            if (r0 == d && r1 > 0) { c.vocab_size = r1; found = true; break; }
            if (r1 == d && r0 > 0) { c.vocab_size = r0; found = true; break; }
        }
        if (!found) throw Error("vocab_size missing; add architecture vocab_size or embeddings tensor");
    }
    // validate, types.rs:181-241
    const std::pair<const char*, uint32_t> nonzero[] = {
        {"embedding_length", c.embedding_length}, {"attention_head_count", c.attention_head_count}, {"block_count", c.block_count},
        {"context_length", c.context_length}, {"feed_forward_length", c.feed_forward_length}, {"vocab_size", c.vocab_size},
        {"attention_head_count_kv", c.attention_head_count_kv}, {"attention_key_length", c.attention_key_length}};
    for (const auto& [name, v] : nonzero)
        if (v == 0) throw Error(std::string(name) + " must be > 0");
    if (c.embedding_length != c.attention_head_count * c.attention_key_length)
        throw Error("embedding_length " + std::to_string(d) + " must equal attention_head_count " +
                    std::to_string(c.attention_head_count) + " * attention_key_length " + std::to_string(c.attention_key_length));
    if (d % c.attention_head_count)
        throw Error("embedding_length " + std::to_string(d) + " not divisible by attention_head_count " + std::to_string(c.attention_head_count));
    if (c.attention_head_count % c.attention_head_count_kv)
        throw Error("attention_head_count " + std::to_string(c.attention_head_count) + " not divisible by attention_head_count_kv " +
                    std::to_string(c.attention_head_count_kv));
    if (!std::isfinite(c.rope_freq_base) || c.rope_freq_base <= 0.0f) throw Error("rope_freq_base must be finite and > 0");
    if (!std::isfinite(c.rope_freq_scale) || c.rope_freq_scale <= 0.0f) throw Error("rope_freq_scale must be finite and > 0");
    return c;
}

using Views = std::map<std::string, TensorView>;

// Bounds of every known-size tensor against the data section first (src/infer/load.rs:41-63), then one view per
// tensor with shape, alignment, dtype and bounds checks (src/infer/tensor_views.rs:29-117).
inline Views build_views(const std::vector<TensorInfo>& tensors, uint64_t weights_len) {
    for (const auto& t : tensors) {
        const DTypeLayout* l = dtype_layout(t.dtype);
        if (!l) continue;
        uint64_t n = 1;
        for (uint64_t dim : t.shape) n *= dim;
        const uint64_t blocks = n / l->block_elems + (n % l->block_elems != 0);
        uint64_t need, end;
        if (mul_overflow(blocks, l->block_bytes, &need)) throw Error("tensor size overflow");
        if (add_overflow(t.offset, need, &end)) end = UINT64_MAX;
        if (end > weights_len)
            throw Error("tensor '" + t.name + "' overflows weights blob: [" + std::to_string(t.offset) + ".." + std::to_string(end) +
                        ") > " + std::to_string(weights_len));
    }
    Views views;
    for (const auto& t : tensors) {
        if (t.shape.empty()) throw Error("tensor '" + t.name + "' has empty shape");
        for (size_t i = 0; i < t.shape.size(); ++i)
            if (t.shape[i] == 0) throw Error("tensor '" + t.name + "' has zero in dimension " + std::to_string(i));
        const uint64_t align = t.dtype == kF16Code ? 2 : t.dtype == kF32Code ? 4 : 1;
        if (align > 1 && t.offset % align)
            throw Error("tensor '" + t.name + "' offset " + std::to_string(t.offset) + " misaligned for " + dtype_name(t.dtype) +
                        " (align " + std::to_string(align) + ")");
        const DTypeLayout* l = dtype_layout(t.dtype);
        if (!l) throw Error("tensor '" + t.name + "' unsupported dtype: " + dtype_name(t.dtype));
        uint64_t n = 1;
        for (uint64_t dim : t.shape)
            if (mul_overflow(n, dim, &n)) throw Error("tensor element count does not fit in usize");
        const uint64_t blocks = n / l->block_elems + (n % l->block_elems != 0);
        uint64_t need, end;
        if (mul_overflow(blocks, l->block_bytes, &need)) throw Error("tensor size overflow");
        if (add_overflow(t.offset, need, &end)) throw Error("tensor end offset overflow");
        if (end > weights_len)
            throw Error("tensor '" + t.name + "' overflows weights blob or starts beyond end (off=" + std::to_string(t.offset) +
                        ", nbytes=" + std::to_string(need) + ", total=" + std::to_string(weights_len) + ")");
        TensorView v;
        v.dtype = t.dtype;
        v.shape = t.shape;
        v.strides.assign(t.shape.size(), 1);
        uint64_t stride = 1;
        for (size_t i = t.shape.size(); i-- > 0;) {
            v.strides[i] = stride;
            stride *= t.shape[i];
        }
        v.byte_offset = t.offset;
        v.nbytes = need;
        views[t.name] = std::move(v);
    }
    return views;
}

// ---- tensor-name mapping, src/infer/mapping.rs ------------------------------------------------------------
inline const std::string* first_present(const Views& views, const std::vector<std::string>& names) {
    for (const auto& n : names)
        if (views.count(n)) return &n;
    return nullptr;
}
inline std::string require_present(const Views& views, const std::vector<std::string>& names) {
    if (const std::string* n = first_present(views, names)) return *n;
    std::string tried;
    for (size_t i = 0; i < names.size(); ++i) tried += (i ? ", " : "") + names[i];
    throw Error("missing required tensor; tried: " + tried);
}
inline void validate_norm_weight(const std::string& label, const TensorView& v, uint64_t dim) {   // mapping.rs:76-91
    if (v.dtype != kF16Code && v.dtype != kF32Code) throw Error(label + " expected F16 or F32, got " + dtype_name(v.dtype));
    if (v.shape.size() != 1 || v.shape[0] != dim)
        throw Error(label + " shape invalid: expected [" + std::to_string(dim) + "], got " + shape_text(v.shape));
}

struct LayerNames {   // tensor chosen for each role; empty string = absent (optional roles only)
    std::string tok_embeddings, wq, wk, wv, bq, bk, bv, wo, w_gate, w_up, w_down, attn_norm, ffn_norm;
    uint64_t d_model = 0, hidden_dim = 0;
};

inline LayerNames map_standard_layer(const Views& views, const Config& cfg, uint64_t layer) {   // mapping.rs:95-353
    LayerNames out;
    out.tok_embeddings = require_present(views, embedding_names());
    const TensorView& tok = views.at(out.tok_embeddings);
    if (tok.dtype != kF16Code && tok.dtype != kQ80Code)
        throw Error("tok_embeddings.weight expected F16 or Q8_0 [*, *], got " + dtype_name(tok.dtype));
    if (tok.shape.size() != 2) throw Error("embeddings shape invalid: expected rank-2, got " + shape_text(tok.shape));
    const uint64_t r0 = tok.shape[0], r1 = tok.shape[1], d = cfg.embedding_length;
    uint64_t vocab_dim;
    if (r1 == d) vocab_dim = r0;        // [vocab, d_model]
    else if (r0 == d) vocab_dim = r1;   // [d_model, vocab]
    else throw Error("embeddings dims " + shape_text(tok.shape) + " do not contain d_model " + std::to_string(d));
    if (cfg.vocab_size != vocab_dim)
        throw Error("vocab_size meta " + std::to_string(cfg.vocab_size) + " != embeddings vocab dim " + std::to_string(vocab_dim) +
                    " (shape=" + shape_text(tok.shape) + ")");
    if (layer >= cfg.block_count)
        throw Error("layer " + std::to_string(layer) + " out of range (block_count=" + std::to_string(cfg.block_count) + ")");
    const std::string L = "layers." + std::to_string(layer) + ".", B = "blk." + std::to_string(layer) + ".";
    auto optional_name = [&](const std::vector<std::string>& names) {
        const std::string* n = first_present(views, names);
        return n ? *n : std::string();
    };
    out.wq = require_present(views, {L + "attention.wq.weight", B + "attn_q.weight"});
    out.wk = require_present(views, {L + "attention.wk.weight", B + "attn_k.weight"});
    out.wv = require_present(views, {L + "attention.wv.weight", B + "attn_v.weight"});
    out.bq = optional_name({L + "attention.wq.bias", B + "attn_q.bias"});
    out.bk = optional_name({L + "attention.wk.bias", B + "attn_k.bias"});
    out.bv = optional_name({L + "attention.wv.bias", B + "attn_v.bias"});
    out.wo = require_present(views, {L + "attention.wo.weight", B + "attn_output.weight"});
    out.w_gate = require_present(views, {L + "feed_forward.w3.weight", B + "ffn_gate.weight"});   // LLaMA: w3 gate, w1 up, w2 down
    out.w_up = require_present(views, {L + "feed_forward.w1.weight", B + "ffn_up.weight"});
    out.w_down = require_present(views, {L + "feed_forward.w2.weight", B + "ffn_down.weight"});
    out.attn_norm = optional_name({L + "attention_norm.weight", L + "attn_norm.weight", B + "attn_norm.weight"});
    out.ffn_norm = optional_name({L + "ffn_norm.weight", L + "feed_forward_norm.weight", B + "ffn_norm.weight"});

    const std::pair<const char*, const std::string*> gemm_roles[] = {{"wq", &out.wq},         {"wk", &out.wk},     {"wv", &out.wv},
                                                                      {"wo", &out.wo},         {"w_gate", &out.w_gate}, {"w_up", &out.w_up},
                                                                      {"w_down", &out.w_down}};
    for (const auto& [role, name] : gemm_roles) {
        const uint32_t dt = views.at(*name).dtype;
        if (dt != kF16Code && dt != kQ51Code) throw Error(std::string("tensor ") + role + " expected F16 or Q5_1, got " + dtype_name(dt));
    }
    auto dim = [&](const std::string& name, size_t i) {
        const auto& s = views.at(name).shape;
        return i < s.size() ? s[i] : 0;
    };
    for (const auto& [role, name] : {gemm_roles[0], gemm_roles[1], gemm_roles[2], gemm_roles[3]})
        if (dim(*name, 0) != d || dim(*name, 1) == 0)
            throw Error(std::string(role) + " shape invalid: expected [d_model, N], got " + shape_text(views.at(*name).shape));
    const uint64_t hd = cfg.attention_key_length, nq = cfg.attention_head_count * hd, nkv = cfg.attention_head_count_kv * hd;
    const std::tuple<const char*, const std::string*, uint64_t> second[] = {
        {"wq", &out.wq, nq}, {"wk", &out.wk, nkv}, {"wv", &out.wv, nkv}, {"wo", &out.wo, d}};
    for (const auto& [role, name, expect] : second)
        if (dim(*name, 1) != expect)
            throw Error(std::string(role) + " second dim " + std::to_string(dim(*name, 1)) + " != expected " + std::to_string(expect));
    const std::tuple<const char*, const std::string*, uint64_t> biases[] = {{"bq", &out.bq, nq}, {"bk", &out.bk, nkv}, {"bv", &out.bv, nkv}};
    for (const auto& [role, name, expect] : biases) {
        if (name->empty()) continue;
        const TensorView& v = views.at(*name);
        if (v.dtype != kF32Code) throw Error(std::string(role) + " expected F32 bias, got " + dtype_name(v.dtype));
        if (v.shape.size() != 1 || v.shape[0] != expect)
            throw Error(std::string(role) + " shape invalid: expected [" + std::to_string(expect) + "], got " + shape_text(v.shape));
    }
    for (const auto& [role, name] : {gemm_roles[4], gemm_roles[5]})
        if (dim(*name, 0) != d || dim(*name, 1) == 0)
            throw Error(std::string(role) + " shape invalid: expected [d_model, H], got " + shape_text(views.at(*name).shape));
    const uint64_t hidden = dim(out.w_up, 1);
    if (dim(out.w_down, 0) != hidden || dim(out.w_down, 1) != d)
        throw Error("w_down shape invalid: expected [hidden_dim, d_model]=[" + std::to_string(hidden) + ", " + std::to_string(d) +
                    "], got " + shape_text(views.at(out.w_down).shape));
    if (cfg.feed_forward_length != hidden)
        throw Error("model_config.feed_forward_length " + std::to_string(cfg.feed_forward_length) + " != inferred hidden_dim " +
                    std::to_string(hidden));
    if (!out.attn_norm.empty()) validate_norm_weight("attention norm", views.at(out.attn_norm), d);
    if (!out.ffn_norm.empty()) validate_norm_weight("ffn norm", views.at(out.ffn_norm), d);
    out.d_model = d;
    out.hidden_dim = hidden;
    return out;
}

struct LmHead {
    std::string name;
    uint64_t d_model = 0, vocab = 0;
    bool tied = false;
};

// A dedicated output tensor [d_model, vocab] in F16 first; else F16 embeddings that already have that layout
// (mapping.rs:360-437).
inline LmHead map_lm_head(const Views& views, const Config& cfg) {
    static const std::vector<std::string> heads = {"output.weight", "lm_head.weight", "output"};
    if (const std::string* n = first_present(views, heads)) {
        const TensorView& t = views.at(*n);
        if (t.dtype != kF16Code) throw Error("lm_head expected F16, got " + dtype_name(t.dtype));
        if (t.shape.size() != 2) throw Error("lm_head shape invalid: expected [d_model, vocab], got " + shape_text(t.shape));
        if (t.shape[0] == 0 || t.shape[1] == 0)
            throw Error("lm_head dims invalid: non-zero [d_model, vocab] required: " + shape_text(t.shape));
        return {*n, t.shape[0], t.shape[1], false};
    }
    if (const std::string* n = first_present(views, embedding_names())) {
        const TensorView& t = views.at(*n);
        if (t.dtype != kF16Code)
            throw Error("tied lm_head requires F16 embeddings when output head is absent; tensor " + *n + " has " + dtype_name(t.dtype));
        if (t.shape.size() != 2)
            throw Error("tied lm_head embedding shape invalid: expected [d_model, vocab], got " + shape_text(t.shape));
        if (t.shape[0] != cfg.embedding_length || t.shape[1] != cfg.vocab_size)
            throw Error("tied lm_head embedding layout unsupported: expected [d_model, vocab]=[" + std::to_string(cfg.embedding_length) +
                        ", " + std::to_string(cfg.vocab_size) + "], got " + shape_text(t.shape));
        return {*n, cfg.embedding_length, cfg.vocab_size, true};
    }
    throw Error(
        "output projection tensor not found; expected one of output.weight, lm_head.weight, output or tied F16 embeddings in "
        "[d_model, vocab] layout");
}

inline std::string map_output_norm(const Views& views, const Config& cfg) {   // mapping.rs:439-459; "" when absent
    static const std::vector<std::string> names = {"output_norm.weight", "norm.weight", "model.norm.weight"};
    const std::string* n = first_present(views, names);
    if (!n) return {};
    validate_norm_weight("output norm", views.at(*n), cfg.embedding_length);
    return *n;
}

inline std::pair<uint64_t, uint64_t> validate_standard_layers(const Views& views, const Config& cfg) {   // mapping.rs:461-493
    if (cfg.block_count == 0) throw Error("model_config.block_count must be > 0");
    uint64_t d = 0, h = 0;
    for (uint32_t layer = 0; layer < cfg.block_count; ++layer) {
        LayerNames w;
        try {
            w = map_standard_layer(views, cfg, layer);
        } catch (const Error& e) {
            throw Error("mapping standard layer " + std::to_string(layer) + ": " + e.what());
        }
        if (layer && d != w.d_model)
            throw Error("layer " + std::to_string(layer) + " d_model mismatch: expected " + std::to_string(d) + ", got " + std::to_string(w.d_model));
        if (layer && h != w.hidden_dim)
            throw Error("layer " + std::to_string(layer) + " hidden_dim mismatch: expected " + std::to_string(h) + ", got " +
                        std::to_string(w.hidden_dim));
        d = w.d_model;
        h = w.hidden_dim;
    }
    return {d, h};
}

// Which way the embedding table is laid out and where one token's values start (src/infer/embeddings.rs:33-60).
// In either orientation a token's d_model values are contiguous: dimension 0 of a GGUF shape is the fastest.
struct EmbeddingRow {
    std::string name;
    uint32_t dtype = 0;
    uint64_t byte_offset = 0, row_bytes = 0, vocab = 0;
};
inline EmbeddingRow embedding_row(const Views& views, const Config& cfg, uint64_t token_id) {
    EmbeddingRow r;
    r.name = require_present(views, embedding_names());
    const TensorView& tok = views.at(r.name);
    if (tok.shape.size() != 2) throw Error("embeddings must be [vocab, d_model]");
    const uint64_t r0 = tok.shape[0], r1 = tok.shape[1], d = cfg.embedding_length, v = cfg.vocab_size;
    const bool rows_are_vocab = v == r0 ? true : v == r1 ? false : r1 == d ? true : r0 == d ? false : (r1 == d);
    r.vocab = rows_are_vocab ? r0 : r1;
    if (token_id >= r.vocab)
        throw Error("token_id " + std::to_string(token_id) + " out of range for vocab size " + std::to_string(r.vocab));
    r.dtype = tok.dtype;
    if (tok.dtype == kF16Code) r.row_bytes = d * 2;
    else if (tok.dtype == kQ80Code) r.row_bytes = (d + 31) / 32 * 34;
    else throw Error("unsupported embedding dtype: " + dtype_name(tok.dtype));
    r.byte_offset = tok.byte_offset + token_id * r.row_bytes;
    if (r.byte_offset + r.row_bytes > tok.byte_offset + tok.nbytes) throw Error("embedding row lies outside its tensor");
    return r;
}

// ---- JSON description of everything above, for bindings and tests ---------------------------------------
inline void json_escape(std::string& out, const std::string& s) {
    out += '"';
    for (unsigned char ch : s) {
        switch (ch) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (ch < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof buf, "\\u%04x", ch);
                    out += buf;
                } else {
                    out += static_cast<char>(ch);
                }
        }
    }
    out += '"';
}
inline void json_scalar(std::string& out, const Scalar& s) {
    char buf[64];
    switch (s.type) {
        case kU8: case kU16: case kU32: case kU64: out += std::to_string(s.u); break;
        case kI8: case kI16: case kI32: case kI64: out += std::to_string(s.i); break;
        case kBool: out += s.u ? "true" : "false"; break;
        case kStr: json_escape(out, s.s); break;
        default:
            if (std::isfinite(s.f)) {
                std::snprintf(buf, sizeof buf, "%.17g", s.f);
                out += buf;
            } else {
                out += "null";
            }
    }
}
inline void json_u64_list(std::string& out, const std::vector<uint64_t>& v) {
    out += '[';
    for (size_t i = 0; i < v.size(); ++i) out += (i ? "," : "") + std::to_string(v[i]);
    out += ']';
}
inline void json_name_or_null(std::string& out, const std::string& s) {
    if (s.empty()) out += "null";
    else json_escape(out, s);
}

constexpr size_t kJsonArrayPreview = 32;   // longer metadata arrays (tokenizer tables) are cut to this many elements

// Everything the host layer derives from one file.  A stage that fails reports "<stage>_error" and the later
// stages that depend on it are left out.
inline std::string describe_json(const Model& m) {
    std::string o = "{\"version\":" + std::to_string(m.version) + ",\"data_offset\":" + std::to_string(m.data_offset) +
                    ",\"file_len\":" + std::to_string(m.file_len) + ",\"metadata\":{";
    bool first = true;
    for (const auto& [key, v] : m.metadata) {
        if (!first) o += ',';
        first = false;
        json_escape(o, key);
        if (v.is_array) {
            o += ":{\"type\":9,\"elem_type\":" + std::to_string(v.elem_type) + ",\"len\":" + std::to_string(v.array.size()) + ",\"value\":[";
            for (size_t i = 0; i < v.array.size() && i < kJsonArrayPreview; ++i) {
                if (i) o += ',';
                json_scalar(o, v.array[i]);
            }
            o += "]}";
        } else {
            o += ":{\"type\":" + std::to_string(v.scalar.type) + ",\"value\":";
            json_scalar(o, v.scalar);
            o += '}';
        }
    }
    o += "},\"tensors\":[";
    for (size_t i = 0; i < m.tensors.size(); ++i) {
        const auto& t = m.tensors[i];
        if (i) o += ',';
        o += "{\"name\":";
        json_escape(o, t.name);
        o += ",\"dtype\":";
        json_escape(o, dtype_name(t.dtype));
        o += ",\"dtype_raw\":" + std::to_string(t.dtype) + ",\"shape\":";
        json_u64_list(o, t.shape);
        o += ",\"offset\":" + std::to_string(t.offset) + '}';
    }
    o += ']';
    std::optional<Config> cfg;
    try {
        cfg = config_from_metadata(m.metadata, m.tensors);
        char buf[160];
        o += ",\"config\":{\"architecture\":";
        json_escape(o, cfg->architecture);
        std::snprintf(buf, sizeof buf, ",\"layer_norm_epsilon\":%.9g,\"rope_freq_base\":%.9g,\"rope_freq_scale\":%.9g",
                      cfg->layer_norm_epsilon, cfg->rope_freq_base, cfg->rope_freq_scale);
        o += ",\"block_count\":" + std::to_string(cfg->block_count) + ",\"context_length\":" + std::to_string(cfg->context_length) +
             ",\"embedding_length\":" + std::to_string(cfg->embedding_length) + ",\"feed_forward_length\":" +
             std::to_string(cfg->feed_forward_length) + ",\"attention_head_count\":" + std::to_string(cfg->attention_head_count) +
             ",\"attention_head_count_kv\":" + std::to_string(cfg->attention_head_count_kv) + ",\"attention_key_length\":" +
             std::to_string(cfg->attention_key_length) + ",\"vocab_size\":" + std::to_string(cfg->vocab_size) + ",\"rope_layout\":" +
             std::to_string(cfg->rope_layout()) + buf + '}';
    } catch (const Error& e) {
        o += ",\"config_error\":";
        json_escape(o, e.what());
    }
    std::optional<Views> views;
    try {
        if (m.data_offset > m.file_len)
            throw Error("GGUF data_offset " + std::to_string(m.data_offset) + " beyond file size " + std::to_string(m.file_len));
        views = build_views(m.tensors, m.file_len - m.data_offset);
        o += ",\"views\":{";
        first = true;
        for (const auto& [name, v] : *views) {
            if (!first) o += ',';
            first = false;
            json_escape(o, name);
            o += ":{\"dtype\":";
            json_escape(o, dtype_name(v.dtype));
            o += ",\"shape\":";
            json_u64_list(o, v.shape);
            o += ",\"strides\":";
            json_u64_list(o, v.strides);
            o += ",\"byte_offset\":" + std::to_string(v.byte_offset) + ",\"nbytes\":" + std::to_string(v.nbytes) + '}';
        }
        o += '}';
    } catch (const Error& e) {
        o += ",\"views_error\":";
        json_escape(o, e.what());
    }
    if (cfg && views) {
        // every layer on its own: a file may hold a subset of the layers its block_count names
        o += ",\"layers\":[";
        for (uint32_t l = 0; l < cfg->block_count; ++l) {
            if (l) o += ',';
            try {
                const LayerNames w = map_standard_layer(*views, *cfg, l);
                std::string layer = "{";
                const std::pair<const char*, const std::string*> roles[] = {
                    {"tok_embeddings", &w.tok_embeddings}, {"wq", &w.wq}, {"wk", &w.wk}, {"wv", &w.wv}, {"bq", &w.bq}, {"bk", &w.bk},
                    {"bv", &w.bv}, {"wo", &w.wo}, {"w_gate", &w.w_gate}, {"w_up", &w.w_up}, {"w_down", &w.w_down},
                    {"attn_norm", &w.attn_norm}, {"ffn_norm", &w.ffn_norm}};
                for (const auto& [role, name] : roles) {
                    layer += std::string("\"") + role + "\":";
                    json_name_or_null(layer, *name);
                    layer += ',';
                }
                o += layer + "\"d_model\":" + std::to_string(w.d_model) + ",\"hidden_dim\":" + std::to_string(w.hidden_dim) + '}';
            } catch (const Error& e) {
                o += "{\"error\":";
                json_escape(o, e.what());
                o += '}';
            }
        }
        o += ']';
        try {
            const LmHead h = map_lm_head(*views, *cfg);
            o += ",\"lm_head\":{\"name\":";
            json_escape(o, h.name);
            o += ",\"d_model\":" + std::to_string(h.d_model) + ",\"vocab\":" + std::to_string(h.vocab) + ",\"tied\":" +
                 (h.tied ? "true" : "false") + '}';
        } catch (const Error& e) {
            o += ",\"lm_head_error\":";
            json_escape(o, e.what());
        }
        try {
            const std::string n = map_output_norm(*views, *cfg);
            o += ",\"output_norm\":";
            json_name_or_null(o, n);
        } catch (const Error& e) {
            o += ",\"output_norm_error\":";
            json_escape(o, e.what());
        }
    }
    return o + '}';
}

}  // namespace gguf
}  // namespace m40host
