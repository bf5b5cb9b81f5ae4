// wrq_loader.hpp -- matrices from a safetensors model file into packed device matrices.  Header
// only, on top of wrq.hpp.
//
// Mirrors the part of the reference's loader that feeds the quantized path:
//   Reader (names / contains / shape / tensor)        src/runtime/loader.rs:44-74
//   Loader::tensor_shape                              src/runtime/loader.rs:389-392 (file order reversed: x fastest)
//   Loader::load_matrix_f16(_discount)                src/runtime/loader.rs:568-621, :651-686
//   Loader::load_matrix, load_matrix_discount         src/runtime/loader.rs:709-762
//   Quant { None, Int8, NF4, SF4 }                    src/runtime/model.rs:122-135
// The discount (2^-(layer / rescale) on att.output and ffn.value) multiplies in f32 and rounds to
// f16 (nearest even, subnormals kept: `half::f16::from_f32`) before the matrix is packed; the loader does
// it on the device, `Loader::discounted` is the same expression on the host.
//   Lora, LoraBlend, lora_matrices, lora_vectors      src/runtime/loader.rs:106-186, :328-386 (adapters blended in at load time:
//                                                     `blend_lora` with alpha / rank for the low-rank halves, `blend` for whole tensors)
//
// The file format (safetensors): 8 bytes little-endian header length N, N bytes of JSON
// `{ name: { "dtype", "shape", "data_offsets": [begin, end] }, "__metadata__": {..} }`, then the
// data; offsets count from the end of the header.  The file is mapped, not read: a tensor's bytes
// go from the page cache to the device in one copy.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <regex>
#include <sstream>

#include "wrq.hpp"

namespace wrq {

struct LoaderError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// f16 <-> f32 on the host, IEEE 754 binary16, round to nearest even, subnormals and specials kept
inline float f16_to_f32(f16 h) {
    const uint32_t sign = (uint32_t)(h.bits & 0x8000) << 16, exp = (h.bits >> 10) & 31, man = h.bits & 0x3ff;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { // subnormal: man * 2^-24
            float v = (float)man * 5.9604644775390625e-8f;
            std::memcpy(&bits, &v, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

inline f16 f16_from_f32(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000);
    const uint32_t abs = x & 0x7fffffffu;
    f16 h;
    if (abs >= 0x7f800000u) { // inf, nan (quiet bit set so that a nan stays one)
        h.bits = sign | 0x7c00 | (abs > 0x7f800000u ? (uint16_t)(0x200 | ((abs >> 13) & 0x3ff)) : 0);
    } else if (abs >= 0x477ff000u) { // rounds to 65520 or more: overflow to infinity
        h.bits = sign | 0x7c00;
    } else if (abs >= 0x38800000u) { // normal range: drop 13 bits, nearest even
        const uint32_t v = abs - 0x38000000u;
        h.bits = sign | (uint16_t)((v + 0xfffu + ((v >> 13) & 1)) >> 13);
    } else if (abs >= 0x33000000u) { // subnormal result: shift the 24-bit significand into place
        const uint32_t e = abs >> 23, m = (abs & 0x7fffffu) | 0x800000u;
        const uint32_t shift = 126 - e; // 14 .. 24
        const uint32_t half = 1u << (shift - 1), rest = m & ((1u << shift) - 1);
        uint32_t q = m >> shift;
        if (rest > half || (rest == half && (q & 1))) q++;
        h.bits = sign | (uint16_t)q;
    } else {
        h.bits = sign;
    }
    return h;
}

// ------------------------------------------------------------------ the model file

class SafeTensors {
  public:
    struct Entry {
        std::string dtype;
        std::vector<uint64_t> shape; // as in the file: slowest axis first
        uint64_t begin = 0, end = 0;
    };

    explicit SafeTensors(const std::string &path) {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) throw LoaderError("cannot open " + path);
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size < 8) {
            ::close(fd_);
            throw LoaderError(path + ": not a safetensors file (shorter than its header length)");
        }
        size_ = (size_t)st.st_size;
        void *p = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (p == MAP_FAILED) {
            ::close(fd_);
            throw LoaderError("cannot map " + path);
        }
        base_ = static_cast<const uint8_t *>(p);
        try {
            uint64_t n = 0;
            for (int i = 7; i >= 0; i--) n = (n << 8) | base_[i];
            if (n > size_ - 8) throw LoaderError(path + ": header of " + std::to_string(n) + " bytes runs past the file");
            data_ = base_ + 8 + n;
            data_size_ = size_ - 8 - n;
            Json js{reinterpret_cast<const char *>(base_ + 8), reinterpret_cast<const char *>(base_ + 8 + n)};
            js.header(entries_, metadata_);
            for (const auto &kv : entries_) {
                const Entry &e = kv.second;
                if (e.end < e.begin || e.end > data_size_) throw LoaderError(kv.first + ": data offsets run past the file");
                // the header is untrusted: extents whose product wraps must not pass as a small tensor
                uint64_t bytes = dtype_size(e.dtype);
                bool wraps = false;
                for (uint64_t d : e.shape) wraps |= __builtin_mul_overflow(bytes, d, &bytes);
                if (wraps || (e.end - e.begin) != bytes) throw LoaderError(kv.first + ": data size does not fit shape and type");
            }
        } catch (...) {
            munmap(const_cast<uint8_t *>(base_), size_);
            ::close(fd_);
            throw;
        }
    }
    ~SafeTensors() {
        munmap(const_cast<uint8_t *>(base_), size_);
        ::close(fd_);
    }
    SafeTensors(const SafeTensors &) = delete;
    SafeTensors &operator=(const SafeTensors &) = delete;

    std::vector<std::string> names() const {
        std::vector<std::string> out;
        for (const auto &kv : entries_) out.push_back(kv.first);
        return out;
    }
    bool contains(const std::string &name) const { return entries_.count(name) != 0; }
    const Entry &entry(const std::string &name) const {
        const auto it = entries_.find(name);
        if (it == entries_.end()) throw LoaderError("tensor `" + name + "` not found");
        return it->second;
    }
    std::vector<uint64_t> shape(const std::string &name) const { return entry(name).shape; }
    // the tensor's bytes inside the mapping (valid while this object lives)
    std::pair<const uint8_t *, size_t> tensor(const std::string &name) const {
        const Entry &e = entry(name);
        return {data_ + e.begin, (size_t)(e.end - e.begin)};
    }
    const std::map<std::string, std::string> &metadata() const { return metadata_; }

    static size_t dtype_size(const std::string &dt) {
        if (dt == "F16" || dt == "BF16" || dt == "I16" || dt == "U16") return 2;
        if (dt == "F32" || dt == "I32" || dt == "U32") return 4;
        if (dt == "F64" || dt == "I64" || dt == "U64") return 8;
        if (dt == "U8" || dt == "I8" || dt == "BOOL" || dt == "F8_E4M3" || dt == "F8_E5M2") return 1;
        throw LoaderError("unknown element type `" + dt + "`");
    }

  private:
    // the subset of JSON a safetensors header uses: objects, arrays, strings, unsigned integers
    struct Json {
        const char *p, *end;
        void ws() {
            while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) p++;
        }
        char peek() {
            ws();
            if (p >= end) throw LoaderError("safetensors header: unexpected end");
            return *p;
        }
        void expect(char c) {
            if (peek() != c) throw LoaderError(std::string("safetensors header: expected `") + c + "`, found `" + *p + "`");
            p++;
        }
        bool accept(char c) {
            if (peek() != c) return false;
            p++;
            return true;
        }
        std::string string() {
            expect('"');
            std::string s;
            while (true) {
                if (p >= end) throw LoaderError("safetensors header: unterminated string");
                const char c = *p++;
                if (c == '"') break;
                if (c != '\\') {
                    s.push_back(c);
                    continue;
                }
                if (p >= end) throw LoaderError("safetensors header: unterminated escape");
                const char e = *p++;
                switch (e) {
                case 'n': s.push_back('\n'); break;
                case 't': s.push_back('\t'); break;
                case 'r': s.push_back('\r'); break;
                case 'b': s.push_back('\b'); break;
                case 'f': s.push_back('\f'); break;
                case 'u': { // \uXXXX, written out as UTF-8 (surrogate pairs are left as two code units)
                    if (end - p < 4) throw LoaderError("safetensors header: short \\u escape");
                    unsigned v = 0;
                    for (int i = 0; i < 4; i++) {
                        const char h = *p++;
                        v = v * 16 + (h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 : h >= 'A' && h <= 'F' ? h - 'A' + 10 : 0);
                    }
                    if (v < 0x80) {
                        s.push_back((char)v);
                    } else if (v < 0x800) {
                        s.push_back((char)(0xc0 | (v >> 6))), s.push_back((char)(0x80 | (v & 63)));
                    } else {
                        s.push_back((char)(0xe0 | (v >> 12))), s.push_back((char)(0x80 | ((v >> 6) & 63))), s.push_back((char)(0x80 | (v & 63)));
                    }
                    break;
                }
                default: s.push_back(e); // \" \\ \/
                }
            }
            return s;
        }
        uint64_t number() {
            ws();
            if (p >= end || *p < '0' || *p > '9') throw LoaderError("safetensors header: expected an unsigned integer");
            uint64_t v = 0;
            while (p < end && *p >= '0' && *p <= '9') v = v * 10 + (uint64_t)(*p++ - '0');
            return v;
        }
        std::vector<uint64_t> numbers() {
            std::vector<uint64_t> out;
            expect('[');
            if (accept(']')) return out;
            do out.push_back(number());
            while (accept(','));
            expect(']');
            return out;
        }
        void header(std::map<std::string, Entry> &entries, std::map<std::string, std::string> &metadata) {
            expect('{');
            if (accept('}')) return;
            do {
                const std::string name = string();
                expect(':');
                expect('{');
                if (name == "__metadata__") {
                    if (!accept('}')) {
                        do {
                            const std::string k = string();
                            expect(':');
                            metadata[k] = string();
                        } while (accept(','));
                        expect('}');
                    }
                    continue;
                }
                Entry e;
                bool dt = false, sh = false, off = false;
                do {
                    const std::string k = string();
                    expect(':');
                    if (k == "dtype") e.dtype = string(), dt = true;
                    else if (k == "shape") e.shape = numbers(), sh = true;
                    else if (k == "data_offsets") {
                        const auto o = numbers();
                        if (o.size() != 2) throw LoaderError(name + ": data_offsets is a pair");
                        e.begin = o[0], e.end = o[1], off = true;
                    } else throw LoaderError(name + ": unknown field `" + k + "`");
                } while (accept(','));
                expect('}');
                if (!dt || !sh || !off) throw LoaderError(name + ": dtype, shape and data_offsets are required");
                entries[name] = e;
            } while (accept(','));
            expect('}');
        }
    };

    int fd_ = -1;
    size_t size_ = 0, data_size_ = 0;
    const uint8_t *base_ = nullptr, *data_ = nullptr;
    std::map<std::string, Entry> entries_;
    std::map<std::string, std::string> metadata_;
};

// --------------------------------------------------------------------- the loader

enum class Quant { None, Int8, NF4, SF4 }; // src/runtime/model.rs:122-135

// Low-rank adapters blended into the weights while they are loaded (src/runtime/loader.rs:106-186).
// A blend pattern is a regular expression over tensor names and a factor; of the patterns of one adapter that match a name,
// the LAST one counts (`rfind`, loader.rs:336-343).
struct LoraBlendPattern {
    std::regex pattern;
    float alpha;
    LoraBlendPattern(const std::string &p, float a) : pattern(p, std::regex::ECMAScript), alpha(a) {}
};

struct LoraBlend : std::vector<LoraBlendPattern> {
    // replaces all vectors, adds to all matrices with `alpha` (loader.rs:120-124)
    static LoraBlend full(float alpha) { return LoraBlend().add_nominal(1.0f).add_matrices(alpha); }
    LoraBlend &add_nominal(float alpha) { // every tensor, interpolated with `alpha` (loader.rs:126-132)
        emplace_back(".+", alpha);
        return *this;
    }
    LoraBlend &add_matrices(float alpha) { // the matrices of the layers (loader.rs:134-145)
        emplace_back("blocks\\.([0-9]+)\\.(att|ffn)\\.(key|value|receptance|gate|output)\\.weight", alpha);
        return *this;
    }
    LoraBlend &add_layer(size_t layer, float alpha) { // ... of one layer (loader.rs:147-160)
        emplace_back("blocks\\." + std::to_string(layer) + "\\.(att|ffn)\\.(key|value|receptance|gate|output)\\.weight", alpha);
        return *this;
    }
    // the factor that applies to `name`, if any pattern matches
    bool factor_of(const std::string &name, float &alpha) const {
        for (auto it = rbegin(); it != rend(); ++it)
            if (std::regex_search(name, it->pattern)) {
                alpha = it->alpha;
                return true;
            }
        return false;
    }
};

struct Lora {
    const SafeTensors *data; // the adapter file; outlives the loader
    LoraBlend blend;
};

class Loader {
  public:
    Loader(const SafeTensors &model, Queue &queue, std::vector<Lora> lora = {}) : model_(model), queue_(queue), lora_(std::move(lora)) {}

    // What `lora_matrices` finds for a matrix name (loader.rs:355-386): per adapter whose last matching pattern gives a
    // factor and whose file holds `<name without .weight>.lora.0` ([?, rank] in the file) and `.lora.1`.
    struct LoraMatrixRef {
        std::string x, y; // tensor names in the adapter file
        const SafeTensors *data;
        uint32_t rank;
        float alpha;
    };
    static std::string lora_stem(const std::string &name) {
        // `name.split('.').filter(|x| !x.contains("weight")).join(".")` (loader.rs:368)
        std::string out, part;
        std::istringstream in(name);
        while (std::getline(in, part, '.'))
            if (part.find("weight") == std::string::npos) out += (out.empty() ? "" : ".") + part;
        return out;
    }
    std::vector<LoraMatrixRef> lora_matrices(const std::string &name) const {
        std::vector<LoraMatrixRef> out;
        for (const Lora &l : lora_) {
            float alpha;
            if (!l.blend.factor_of(name, alpha)) continue;
            const std::string stem = lora_stem(name);
            const std::string x = stem + ".lora.0", y = stem + ".lora.1";
            if (!l.data->contains(x) || !l.data->contains(y)) continue;
            const auto shape = l.data->shape(x);
            if (shape.size() < 2 || shape[1] == 0 || shape[1] > 0xffffffffull) throw LoaderError("`" + x + "`: an adapter half has two axes");
            out.push_back(LoraMatrixRef{x, y, l.data, (uint32_t)shape[1], alpha});
        }
        return out;
    }
    // ... and `lora_vectors` (loader.rs:330-353): a tensor of the same name in the adapter file
    struct LoraVectorRef {
        const SafeTensors *data;
        float alpha;
    };
    std::vector<LoraVectorRef> lora_vectors(const std::string &name) const {
        std::vector<LoraVectorRef> out;
        for (const Lora &l : lora_) {
            float alpha;
            if (l.blend.factor_of(name, alpha) && l.data->contains(name)) out.push_back(LoraVectorRef{l.data, alpha});
        }
        return out;
    }

    // src/runtime/loader.rs:389-392 and `Shape::from_slice_rev`: [out, in] in the file is [in, out, 1, 1] here
    Shape tensor_shape(const std::string &name) const { return shape_of(model_, name); }

    // src/runtime/loader.rs:568-592: the file's matrix, then every adapter blended in on the device
    // (`blend_lora` with factor alpha / rank for the low-rank halves, `blend` with alpha for a tensor of the same name)
    TensorGpu<f16> load_matrix_f16(const std::string &name) const {
        TensorGpu<f16> t = upload_f16(model_, name);
        blend_adapters(t, name, 1.0f);
        return t;
    }
    // src/runtime/loader.rs:594-621, :651-686: x -> f16(discount * f32(x))
    // The file's bytes go to the device as they are and the discount is applied there (`TensorOp::affine`
    // multiplies in f32 and rounds to f16 like the host expression): a host loop over the elements would
    // bound the load at under 1 GB/s against 20+ GB/s for the copy.
    // The adapters join the discounted matrix with factors discount * alpha (/ rank), as in the reference (loader.rs:605-617).
    TensorGpu<f16> load_matrix_f16_discount(const std::string &name, float discount) const {
        TensorGpu<f16> t = upload_f16(model_, name);
        queue_.submit(TensorOp::affine(t, discount, 0.0f));
        blend_adapters(t, name, discount);
        return t;
    }
    // the same values computed on the host (no device): the reference expression, element by element
    std::vector<f16> discounted(const std::string &name, float discount) const {
        const auto bytes = f16_bytes(name);
        std::vector<f16> host(bytes.second / 2);
        std::memcpy(host.data(), bytes.first, bytes.second);
        for (f16 &h : host) h = f16_from_f32(discount * f16_to_f32(h));
        return host;
    }

    // src/runtime/loader.rs:709-733
    Matrix load_matrix(const std::string &name, Quant quant) const { return pack(load_matrix_f16(name), quant); }
    // src/runtime/loader.rs:735-762
    Matrix load_matrix_discount(const std::string &name, Quant quant, float discount) const {
        return pack(load_matrix_f16_discount(name, discount), quant);
    }

  private:
    std::pair<const uint8_t *, size_t> f16_bytes(const std::string &name) const { return f16_bytes_of(model_, name); }
    static std::pair<const uint8_t *, size_t> f16_bytes_of(const SafeTensors &file, const std::string &name) {
        if (file.entry(name).dtype != "F16") // `TensorCpu::<f16>::from_reader`: TensorErrorKind::Type
            throw TensorError(WRQ_ERR_TYPE, "`" + name + "`: data type mismatch (" + file.entry(name).dtype + ", expected F16)");
        return file.tensor(name);
    }
    static Shape shape_of(const SafeTensors &file, const std::string &name) {
        const auto s = file.shape(name);
        if (s.empty() || s.size() > 4) throw LoaderError("`" + name + "`: " + std::to_string(s.size()) + " axes (1 to 4 are tensors)");
        uint32_t d[4] = {1, 1, 1, 1};
        for (size_t i = 0; i < s.size(); i++) {
            if (s[s.size() - 1 - i] > 0xffffffffull) throw LoaderError("`" + name + "`: extent beyond 32 bits");
            d[i] = (uint32_t)s[s.size() - 1 - i];
        }
        return Shape(d[0], d[1], d[2], d[3]);
    }
    static TensorGpu<f16> upload_f16(const SafeTensors &file, const std::string &name) {
        const auto bytes = f16_bytes_of(file, name);
        TensorGpu<f16> t = TensorGpu<f16>::init(shape_of(file, name));
        if (hipMemcpy(t.data(), bytes.first, bytes.second, hipMemcpyHostToDevice) != hipSuccess) throw TensorError(WRQ_ERR_DEVICE, "hipMemcpy failed");
        return t;
    }
    void blend_adapters(const TensorGpu<f16> &t, const std::string &name, float scale) const {
        for (const LoraMatrixRef &l : lora_matrices(name)) {
            const TensorGpu<float> factor = TensorGpu<float>::from_data(Shape(4, 1, 1, 1), {scale * l.alpha / (float)l.rank, 1.0f, 0.0f, 0.0f});
            const TensorGpu<f16> x = upload_f16(*l.data, l.x), y = upload_f16(*l.data, l.y);
            queue_.submit(TensorOp::blend_lora(factor, TensorGpuView<f16>(x), TensorGpuView<f16>(y), TensorGpuView<f16>(t)));
            queue_.sync(); // the adapter halves and the factor are released here
        }
        for (const LoraVectorRef &l : lora_vectors(name)) {
            const TensorGpu<float> factor = TensorGpu<float>::from_data(Shape(4, 1, 1, 1), {scale * l.alpha, 1.0f, 0.0f, 0.0f});
            const TensorGpu<f16> v = upload_f16(*l.data, name);
            queue_.submit(TensorOp::blend(factor, v, t));
            queue_.sync();
        }
    }
    Matrix pack(const TensorGpu<f16> &buffer, Quant quant) const {
        switch (quant) {
        case Quant::None: return Matrix::fp16(buffer);
        case Quant::Int8: return Matrix::quant_u8(buffer, queue_);
        case Quant::NF4: return Matrix::quant_nf4(buffer, queue_);
        case Quant::SF4: return Matrix::quant_sf4(buffer, queue_, 5.0);
        }
        throw LoaderError("unknown quantization");
    }
    const SafeTensors &model_;
    Queue &queue_;
    std::vector<Lora> lora_;
};

} // namespace wrq
