// Element types, dynamically typed scalars and host tensors.
// Mirrors kn-graph/src/dtype.rs (DType :24-37, DScalar :56-69, DTensor :41-54, Specials :79-85)
// and adds F16, which the reference IR lacks, for half-precision storage with f32 accumulation.
#pragma once

#include <cmath>
#include <cstring>
#include <memory>

#include "common.h"

namespace kn {

// The numeric codes are part of the serialised graph format and the C ABI.
enum class DType : uint8_t {
    F32 = 0,
    F64 = 1,
    I8 = 2,
    I16 = 3,
    I32 = 4,
    I64 = 5,
    U8 = 6,
    U16 = 7,
    U32 = 8,
    U64 = 9,
    Bool = 10,
    F16 = 11,
};
constexpr int DTYPE_COUNT = 12;

inline bool dtype_valid(int code) { return code >= 0 && code < DTYPE_COUNT; }

inline size_t dtype_bytes(DType t) {
    switch (t) {
        case DType::F32: case DType::I32: case DType::U32: return 4;
        case DType::F64: case DType::I64: case DType::U64: return 8;
        case DType::I16: case DType::U16: case DType::F16: return 2;
        case DType::I8: case DType::U8: case DType::Bool: return 1;
    }
    fail("invalid dtype");
}

inline bool dtype_is_float(DType t) { return t == DType::F32 || t == DType::F64 || t == DType::F16; }
inline bool dtype_is_bool(DType t) { return t == DType::Bool; }
inline bool dtype_is_int(DType t) { return !dtype_is_float(t) && !dtype_is_bool(t); }
inline bool dtype_is_signed(DType t) {
    return dtype_is_float(t) || t == DType::I8 || t == DType::I16 || t == DType::I32 || t == DType::I64;
}

inline const char *dtype_name(DType t) {
    static const char *names[] = {"f32", "f64", "i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "bool", "f16"};
    return names[(int) t];
}

// The spelling of the element type inside generated device code (dtype.rs:150-164); bool is stored as one byte.
inline const char *dtype_c_name(DType t) {
    static const char *names[] = {"float", "double", "int8_t", "int16_t", "int32_t", "int64_t",
                                  "uint8_t", "uint16_t", "uint32_t", "uint64_t", "bool", "_Float16"};
    return names[(int) t];
}

// ---- half precision helpers (round to nearest even), used on the host only
inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mant = x & 0x007fffffu;
    int32_t exp = (int32_t) ((x >> 23) & 0xff);
    if (exp == 0xff) return (uint16_t) (sign | 0x7c00u | (mant ? 0x200u | (mant >> 13) : 0));
    exp = exp - 127 + 15;
    if (exp >= 0x1f) return (uint16_t) (sign | 0x7c00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t) sign;
        mant |= 0x00800000u;
        uint32_t shift = (uint32_t) (14 - exp);
        uint32_t half = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t) (sign | half);
    }
    uint32_t half = ((uint32_t) exp << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t) (sign | half);
}

inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t) h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t mant = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (mant == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                e++;
                mant <<= 1;
            } while (!(mant & 0x400u));
            x = sign | ((uint32_t) (127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 0x1f) {
        x = sign | 0x7f800000u | (mant << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// A single dynamically typed value (dtype.rs:56-69). Floats compare and hash by value with all NaNs
// equal and -0 == +0, which is what makes NaN constants deduplicate in the graph.
struct DScalar {
    DType dtype = DType::F32;
    union {
        double f;    // F32 (exactly representable), F64 and F16 values
        int64_t i;   // signed integers
        uint64_t u;  // unsigned integers and bool
    };

    DScalar() : f(0) {}

    static DScalar f32(float v) { DScalar s; s.dtype = DType::F32; s.f = v; return s; }
    static DScalar f64(double v) { DScalar s; s.dtype = DType::F64; s.f = v; return s; }
    static DScalar f16(float v) { DScalar s; s.dtype = DType::F16; s.f = f16_bits_to_f32(f32_to_f16_bits(v)); return s; }
    static DScalar boolean(bool v) { DScalar s; s.dtype = DType::Bool; s.u = v ? 1 : 0; return s; }
    static DScalar sint(DType t, int64_t v) { DScalar s; s.dtype = t; s.i = v; return s; }
    static DScalar uint(DType t, uint64_t v) { DScalar s; s.dtype = t; s.u = v; return s; }

    bool is_float() const { return dtype_is_float(dtype); }
    bool is_signed_int() const { return dtype_is_int(dtype) && dtype_is_signed(dtype); }

    bool operator==(const DScalar &o) const {
        if (dtype != o.dtype) return false;
        if (is_float()) return (std::isnan(f) && std::isnan(o.f)) || f == o.f;
        if (is_signed_int()) return i == o.i;
        return u == o.u;
    }
    bool operator!=(const DScalar &o) const { return !(*this == o); }

    // Read one element of type `t` from memory / write this value to memory.
    static DScalar load(DType t, const void *p);
    void store(void *p) const;

    // dtype.rs:323-353 value_cast and :355-391 bit_cast
    DScalar value_cast(DType to) const;
    bool bit_cast(DType to, DScalar *out) const;

    // dtype.rs:307-321: the literal used when a single-valued constant is inlined into device code.
    std::string to_c_str() const;
    std::string to_string() const;
};

struct Specials {
    DScalar zero, one, min, max;
};
Specials dtype_specials(DType t);  // dtype.rs:134-148

// Dense, row-major host tensor (the role of DTensor, dtype.rs:41-54).
struct HostTensor {
    DType dtype = DType::F32;
    std::vector<size_t> shape;
    std::shared_ptr<std::vector<uint8_t>> data;

    HostTensor() = default;
    HostTensor(DType dtype, std::vector<size_t> shape);  // zero filled
    HostTensor(DType dtype, std::vector<size_t> shape, const void *src);

    size_t len() const {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        return n;
    }
    size_t rank() const { return shape.size(); }
    size_t nbytes() const { return len() * dtype_bytes(dtype); }
    const uint8_t *bytes() const { return data->data(); }
    uint8_t *bytes_mut() { return data->data(); }
    DScalar at(size_t flat) const { return DScalar::load(dtype, bytes() + flat * dtype_bytes(dtype)); }
    void set(size_t flat, const DScalar &s) { s.store(bytes_mut() + flat * dtype_bytes(dtype)); }

    HostTensor reshape(std::vector<size_t> new_shape) const;
    // dtype.rs:593-619: equal shape, dtype and elements (float-aware)
    bool equals(const HostTensor &o) const;
    // dtype.rs:621-645: shape, dtype and the first 8 elements
    uint64_t hash() const;

    static HostTensor scalar(const DScalar &s);
};

}  // namespace kn
