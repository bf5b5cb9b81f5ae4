// wrq_serde.hpp -- packed matrices to and from the reference's on-disk form.  Header only, on
// top of wrq.hpp.
//
// The reference writes a model with serde into CBOR (the `cbor4ii` crate with its `serde1`
// feature, Cargo.toml:72; examples/serde.rs:234-262).  What serde derives for the types on
// this path:
//   Shape([usize; 4])                          src/tensor/shape.rs:98-99      newtype of a 4-tuple
//   TensorBlob { shape, data (serde_bytes) }   src/tensor/serialization.rs:11-17; every TensorGpu is
//                                              written as the blob of its read-back bytes (:68-76)
//   Matrix::Fp16(t) | Int8 { w, m } | Fp4 { q, w, m }, externally tagged, `Nf4` accepted for `Fp4`
//                                              src/tensor/matrix.rs:80-94
// and how that data model lands in CBOR (RFC 8949): a struct is a definite-length map from
// field names (text strings, declaration order) to values, an enum variant with fields a
// one-entry map from the variant's name to its content, a newtype its content, a tuple a
// definite-length array, `usize` an unsigned integer in its shortest form, serde_bytes a
// definite-length byte string.  So an Int8 matrix is
//   { "Int8": { "w": { "shape": [K, R, B, 1], "data": h'..' }, "m": { "shape": [n, 1, 1, 1], "data": h'..' } } }
// The CBOR items are pinned by the RFC's own examples (tests/cpp/test_host.cpp); the mapping from
// serde to CBOR is the crate's, which is not vendored with the reference and could not be run:
// byte parity with a file the reference wrote is unpinned.  The reader therefore accepts every
// well-formed spelling of the same structure (indefinite-length maps and arrays, integers in
// longer than shortest form, fields in any order, `Nf4`).
#pragma once

#include "wrq.hpp"

namespace wrq {
namespace serde {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ------------------------------------------------------------------ CBOR items (RFC 8949, 3.1)

class Writer {
  public:
    std::vector<uint8_t> out;
    void uint(uint64_t v) { head(0, v); }
    void bytes(const uint8_t *p, size_t n) {
        head(2, n);
        out.insert(out.end(), p, p + n);
    }
    void text(const std::string &s) {
        head(3, s.size());
        out.insert(out.end(), s.begin(), s.end());
    }
    void array(uint64_t n) { head(4, n); }
    void map(uint64_t n) { head(5, n); }

  private:
    void head(int major, uint64_t v) { // shortest form of the argument
        const uint8_t m = (uint8_t)(major << 5);
        int extra = v < 24 ? 0 : v <= 0xff ? 1 : v <= 0xffff ? 2 : v <= 0xffffffffull ? 4 : 8;
        if (extra == 0) {
            out.push_back(m | (uint8_t)v);
            return;
        }
        out.push_back(m | (uint8_t)(extra == 1 ? 24 : extra == 2 ? 25 : extra == 4 ? 26 : 27));
        for (int i = extra - 1; i >= 0; i--) out.push_back((uint8_t)(v >> (8 * i)));
    }
};

class Reader {
  public:
    Reader(const uint8_t *p, size_t n) : p_(p), end_(p + n) {}
    size_t remaining() const { return (size_t)(end_ - p_); }
    // head of the next item: major type, argument; `indefinite` for the open-ended forms
    struct Head {
        int major;
        uint64_t arg;
        bool indefinite;
    };
    Head head() {
        const uint8_t b = byte();
        const int major = b >> 5, info = b & 31;
        if (info < 24) return {major, (uint64_t)info, false};
        if (info == 31) {
            if (major < 2 || major > 5) throw Error("cbor: indefinite length on major type " + std::to_string(major));
            return {major, 0, true};
        }
        if (info > 27) throw Error("cbor: reserved additional information " + std::to_string(info));
        const int extra = 1 << (info - 24);
        uint64_t v = 0;
        for (int i = 0; i < extra; i++) v = (v << 8) | byte();
        return {major, v, false};
    }
    bool at_break() {
        if (p_ >= end_) throw Error("cbor: input ends inside an item");
        if (*p_ != 0xff) return false;
        p_++;
        return true;
    }
    uint64_t uint() {
        const Head h = head();
        if (h.major != 0) throw Error("cbor: expected an unsigned integer, found major type " + std::to_string(h.major));
        return h.arg;
    }
    std::string text() {
        const Head h = head();
        if (h.major != 3 || h.indefinite) throw Error("cbor: expected a definite-length text string");
        const uint8_t *s = take(h.arg);
        return std::string(reinterpret_cast<const char *>(s), (size_t)h.arg);
    }
    std::vector<uint8_t> bytes() {
        const Head h = head();
        if (h.major != 2 || h.indefinite) throw Error("cbor: expected a definite-length byte string");
        const uint8_t *s = take(h.arg);
        return std::vector<uint8_t>(s, s + h.arg);
    }
    // calls `item(index)` for every element of an array, `entry()` for every pair of a map
    template <typename F>
    uint64_t each(int major, const char *what, F &&item) {
        const Head h = head();
        if (h.major != major) throw Error(std::string("cbor: expected ") + what + ", found major type " + std::to_string(h.major));
        uint64_t n = 0;
        if (h.indefinite) {
            while (!at_break()) item(n++);
        } else {
            for (; n < h.arg; n++) item(n);
        }
        return n;
    }

  private:
    uint8_t byte() {
        if (p_ >= end_) throw Error("cbor: input ends inside an item");
        return *p_++;
    }
    const uint8_t *take(uint64_t n) {
        if (n > remaining()) throw Error("cbor: string of " + std::to_string(n) + " bytes runs past the input");
        const uint8_t *s = p_;
        p_ += n;
        return s;
    }
    const uint8_t *p_, *end_;
};

// -------------------------------------------------------------- the blobs (host memory only)

// TensorBlob (src/tensor/serialization.rs:11-17): the shape and the tensor's bytes as they lie in memory.
struct TensorBlob {
    Shape shape;
    std::vector<uint8_t> data;
    bool operator==(const TensorBlob &o) const { return shape == o.shape && data == o.data; }
};

// A Matrix read back to the host: the tensors of its variant, in the variant's field order.
struct MatrixBlob {
    Matrix::Kind kind = Matrix::Kind::Int8;
    TensorBlob w; // Fp16: the f16 weights; Int8 / Fp4: the packed bytes
    TensorBlob m; // Int8: (min, max) f16 pairs; Fp4: absmax f16
    TensorBlob q; // Fp4: the 16 f32 table values
    bool operator==(const MatrixBlob &o) const { return kind == o.kind && w == o.w && m == o.m && q == o.q; }
};

inline void write(Writer &wr, const TensorBlob &t) {
    wr.map(2);
    wr.text("shape");
    wr.array(4);
    for (int i = 0; i < 4; i++) wr.uint(t.shape[i]);
    wr.text("data");
    wr.bytes(t.data.data(), t.data.size());
}

inline void write(Writer &wr, const MatrixBlob &mb) {
    wr.map(1);
    switch (mb.kind) {
    case Matrix::Kind::Fp16:
        wr.text("Fp16");
        write(wr, mb.w);
        break;
    case Matrix::Kind::Int8:
        wr.text("Int8");
        wr.map(2);
        wr.text("w"), write(wr, mb.w);
        wr.text("m"), write(wr, mb.m);
        break;
    case Matrix::Kind::Fp4:
        wr.text("Fp4");
        wr.map(3);
        wr.text("q"), write(wr, mb.q);
        wr.text("w"), write(wr, mb.w);
        wr.text("m"), write(wr, mb.m);
        break;
    }
}

inline TensorBlob read_tensor(Reader &rd, size_t elem_size) {
    TensorBlob t;
    bool has_shape = false, has_data = false;
    rd.each(5, "a map (TensorBlob)", [&](uint64_t) {
        const std::string key = rd.text();
        if (key == "shape") {
            uint32_t d[4] = {1, 1, 1, 1};
            const uint64_t n = rd.each(4, "an array (Shape)", [&](uint64_t i) {
                const uint64_t v = rd.uint();
                if (i >= 4 || v > 0xffffffffull) throw Error("TensorBlob: shape is four 32-bit extents");
                d[i] = (uint32_t)v;
            });
            if (n != 4) throw Error("TensorBlob: shape has " + std::to_string(n) + " extents, expected 4");
            t.shape = Shape(d[0], d[1], d[2], d[3]);
            has_shape = true;
        } else if (key == "data") {
            t.data = rd.bytes();
            has_data = true;
        } else {
            throw Error("TensorBlob: unknown field `" + key + "`");
        }
    });
    if (!has_shape || !has_data) throw Error("TensorBlob: missing field `" + std::string(has_shape ? "data" : "shape") + "`");
    // TensorGpu::from_data_u8: the bytes must fill the shape
    {
        // extents come from the file: a product that wraps must not pass as a small tensor
        uint64_t bytes = elem_size;
        bool wraps = false;
        for (int i = 0; i < 4; i++) wraps |= __builtin_mul_overflow(bytes, (uint64_t)t.shape[i], &bytes);
        if (wraps || t.data.size() != bytes)
            throw Error("TensorBlob: data size not match: " + std::to_string(t.data.size()) + " vs. " + (wraps ? std::string("more than 2^64") : std::to_string(bytes)));
    }
    return t;
}

inline MatrixBlob read_matrix(Reader &rd) {
    MatrixBlob mb;
    const uint64_t n = rd.each(5, "a map (Matrix)", [&](uint64_t index) {
        if (index > 0) throw Error("Matrix: more than one variant");
        const std::string variant = rd.text();
        if (variant == "Fp16") {
            mb.kind = Matrix::Kind::Fp16;
            mb.w = read_tensor(rd, 2);
            return;
        }
        const bool int8 = variant == "Int8";
        if (!int8 && variant != "Fp4" && variant != "Nf4") throw Error("Matrix: unknown variant `" + variant + "`");
        mb.kind = int8 ? Matrix::Kind::Int8 : Matrix::Kind::Fp4;
        bool hw = false, hm = false, hq = false;
        rd.each(5, "a map (the variant's fields)", [&](uint64_t) {
            const std::string key = rd.text();
            if (key == "w") mb.w = read_tensor(rd, 1), hw = true;
            else if (key == "m") mb.m = read_tensor(rd, 2), hm = true;
            else if (key == "q" && !int8) mb.q = read_tensor(rd, 4), hq = true;
            else throw Error("Matrix::" + variant + ": unknown field `" + key + "`");
        });
        if (!hw || !hm || (!int8 && !hq)) throw Error("Matrix::" + variant + ": missing field");
    });
    if (n != 1) throw Error("Matrix: expected one variant");
    // the shapes the products check (src/tensor/ops.rs:809-812, :910-912)
    if (mb.kind == Matrix::Kind::Int8) {
        if (mb.m.shape.len() != (mb.w.shape.len() * 2 + TensorOp::INT8_BLOCK_SIZE - 1) / TensorOp::INT8_BLOCK_SIZE)
            throw Error("Matrix::Int8: " + std::to_string(mb.m.shape.len()) + " scale values for " + std::to_string(mb.w.shape.len()) + " weights");
    } else if (mb.kind == Matrix::Kind::Fp4) {
        if (mb.m.shape.len() != (mb.w.shape.len() * 2 + TensorOp::NF4_BLOCK_SIZE - 1) / TensorOp::NF4_BLOCK_SIZE)
            throw Error("Matrix::Fp4: " + std::to_string(mb.m.shape.len()) + " scale values for " + std::to_string(mb.w.shape.len() * 2) + " weights");
        if (mb.q.shape.len() != 16) throw Error("Matrix::Fp4: the table has 16 entries");
    }
    return mb;
}

inline std::vector<uint8_t> to_vec(const MatrixBlob &mb) {
    Writer wr;
    write(wr, mb);
    return std::move(wr.out);
}

inline MatrixBlob from_slice(const uint8_t *p, size_t n) {
    Reader rd(p, n);
    MatrixBlob mb = read_matrix(rd);
    if (rd.remaining()) throw Error("Matrix: " + std::to_string(rd.remaining()) + " bytes after the value");
    return mb;
}

// ------------------------------------------------------------------- device <-> blob

namespace detail {
template <typename T>
TensorBlob back(const TensorGpu<T> &t) { // `back_in_place`, src/tensor/serialization.rs:74
    const std::vector<T> host = t.back();
    TensorBlob b{t.shape(), std::vector<uint8_t>(host.size() * sizeof(T))};
    std::memcpy(b.data.data(), host.data(), b.data.size());
    return b;
}
template <typename T>
TensorGpu<T> load(const TensorBlob &b) { // `from_data_u8`, src/tensor/serialization.rs:151
    std::vector<T> host(b.data.size() / sizeof(T));
    std::memcpy(host.data(), b.data.data(), b.data.size());
    return TensorGpu<T>::from_data(b.shape, host);
}
} // namespace detail

// Reads the matrix's tensors back (synchronous; the stream that packed them must have finished).
inline MatrixBlob to_blob(const Matrix &mx) {
    MatrixBlob mb;
    mb.kind = mx.kind;
    if (mx.kind == Matrix::Kind::Fp16) {
        mb.w = detail::back(mx.h);
        return mb;
    }
    mb.w = detail::back(mx.w);
    mb.m = detail::back(mx.m);
    if (mx.kind == Matrix::Kind::Fp4) mb.q = detail::back(mx.q);
    return mb;
}

inline Matrix from_blob(const MatrixBlob &mb) {
    if (mb.kind == Matrix::Kind::Fp16) return Matrix::fp16(detail::load<f16>(mb.w));
    if (mb.kind == Matrix::Kind::Int8) return Matrix{Matrix::Kind::Int8, detail::load<uint8_t>(mb.w), detail::load<f16>(mb.m), {}, {}};
    return Matrix{Matrix::Kind::Fp4, detail::load<uint8_t>(mb.w), detail::load<f16>(mb.m), detail::load<float>(mb.q), {}};
}

inline std::vector<uint8_t> to_vec(const Matrix &mx) { return to_vec(to_blob(mx)); }
inline Matrix matrix_from_slice(const uint8_t *p, size_t n) { return from_blob(from_slice(p, n)); }

} // namespace serde
} // namespace wrq
