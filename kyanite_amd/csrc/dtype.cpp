#include "dtype.h"

#include <cinttypes>
#include <limits>

namespace kn {

DScalar DScalar::load(DType t, const void *p) {
    switch (t) {
        case DType::F32: { float v; std::memcpy(&v, p, 4); return DScalar::f32(v); }
        case DType::F64: { double v; std::memcpy(&v, p, 8); return DScalar::f64(v); }
        case DType::F16: {
            uint16_t v; std::memcpy(&v, p, 2);
            DScalar s; s.dtype = DType::F16; s.f = f16_bits_to_f32(v); return s;
        }
        case DType::I8: { int8_t v; std::memcpy(&v, p, 1); return sint(t, v); }
        case DType::I16: { int16_t v; std::memcpy(&v, p, 2); return sint(t, v); }
        case DType::I32: { int32_t v; std::memcpy(&v, p, 4); return sint(t, v); }
        case DType::I64: { int64_t v; std::memcpy(&v, p, 8); return sint(t, v); }
        case DType::U8: { uint8_t v; std::memcpy(&v, p, 1); return uint(t, v); }
        case DType::U16: { uint16_t v; std::memcpy(&v, p, 2); return uint(t, v); }
        case DType::U32: { uint32_t v; std::memcpy(&v, p, 4); return uint(t, v); }
        case DType::U64: { uint64_t v; std::memcpy(&v, p, 8); return uint(t, v); }
        case DType::Bool: { uint8_t v; std::memcpy(&v, p, 1); return boolean(v != 0); }
    }
    fail("invalid dtype");
}

void DScalar::store(void *p) const {
    switch (dtype) {
        case DType::F32: { float v = (float) f; std::memcpy(p, &v, 4); return; }
        case DType::F64: { std::memcpy(p, &f, 8); return; }
        case DType::F16: { uint16_t v = f32_to_f16_bits((float) f); std::memcpy(p, &v, 2); return; }
        case DType::I8: { int8_t v = (int8_t) i; std::memcpy(p, &v, 1); return; }
        case DType::I16: { int16_t v = (int16_t) i; std::memcpy(p, &v, 2); return; }
        case DType::I32: { int32_t v = (int32_t) i; std::memcpy(p, &v, 4); return; }
        case DType::I64: { std::memcpy(p, &i, 8); return; }
        case DType::U8: { uint8_t v = (uint8_t) u; std::memcpy(p, &v, 1); return; }
        case DType::U16: { uint16_t v = (uint16_t) u; std::memcpy(p, &v, 2); return; }
        case DType::U32: { uint32_t v = (uint32_t) u; std::memcpy(p, &v, 4); return; }
        case DType::U64: { std::memcpy(p, &u, 8); return; }
        case DType::Bool: { uint8_t v = u ? 1 : 0; std::memcpy(p, &v, 1); return; }
    }
}

// The low 64 bits of `x as i128` in Rust semantics: truncate toward zero, saturate at the i128 bounds, NaN -> 0.
static uint64_t float_to_i128_low64(double x) {
    if (std::isnan(x)) return 0;
    const double two63 = 9223372036854775808.0;
    const double two127 = 170141183460469231731687303715884105728.0;
    if (x >= two127) return ~0ull;  // i128::MAX
    if (x < -two127) return 0;      // i128::MIN
    double t = std::trunc(x);
    if (t > -two63 && t < two63) return (uint64_t) (int64_t) t;
    // |t| in [2^63, 2^127): an integer m * 2^e with m below 2^53, so the low 64 bits are a shifted mantissa
    int e;
    double m = std::frexp(std::fabs(t), &e);  // |t| = m * 2^e, m in [0.5, 1)
    uint64_t mant = (uint64_t) std::ldexp(m, 53);
    int shift = e - 53;
    uint64_t low = shift >= 64 ? 0 : (mant << shift);
    return t < 0 ? (uint64_t) (0 - low) : low;
}

DScalar DScalar::value_cast(DType to) const {
    // dtype.rs:323-353: go through a wide float and a wide integer, then narrow with wrapping
    double yf;
    uint64_t yi_low;  // low 64 bits of the i128 intermediate
    bool yi_nonzero;
    if (is_float()) {
        yf = f;
        yi_low = float_to_i128_low64(f);
        yi_nonzero = !std::isnan(f) && std::trunc(f) != 0;
    } else if (is_signed_int()) {
        yf = (double) i;
        yi_low = (uint64_t) i;
        yi_nonzero = i != 0;
    } else {
        yf = (double) u;
        yi_low = u;
        yi_nonzero = u != 0;
    }
    switch (to) {
        case DType::F32: return DScalar::f32((float) yf);
        case DType::F64: return DScalar::f64(yf);
        case DType::F16: return DScalar::f16((float) yf);
        case DType::I8: return sint(to, (int8_t) yi_low);
        case DType::I16: return sint(to, (int16_t) yi_low);
        case DType::I32: return sint(to, (int32_t) yi_low);
        case DType::I64: return sint(to, (int64_t) yi_low);
        case DType::U8: return uint(to, (uint8_t) yi_low);
        case DType::U16: return uint(to, (uint16_t) yi_low);
        case DType::U32: return uint(to, (uint32_t) yi_low);
        case DType::U64: return uint(to, yi_low);
        case DType::Bool: return boolean(yf != 0.0 || yi_nonzero);
    }
    fail("invalid dtype");
}

bool DScalar::bit_cast(DType to, DScalar *out) const {
    if (dtype_bytes(dtype) != dtype_bytes(to)) return false;
    if (dtype == DType::Bool || to == DType::Bool) return false;
    uint8_t buf[8] = {0};
    store(buf);
    *out = load(to, buf);
    return true;
}

static std::string c_float_str(double v) {
    // dtype.rs:702-716 DisplayCFloat
    const char *s = std::signbit(v) ? "-" : "";
    if (std::isnan(v)) return std::string("(") + s + "(0.0/0.0))";
    if (std::isinf(v)) return std::string("(") + s + "(1.0/0.0))";
    if (v == 0.0) return std::string("(") + s + "0.0)";
    char buf[64];
    snprintf(buf, sizeof buf, "%.17g", v);
    std::string r = buf;
    // make sure the literal is a floating literal
    if (r.find_first_of(".eEn") == std::string::npos) r += ".0";
    return r;
}

std::string DScalar::to_c_str() const {
    char buf[64];
    switch (dtype) {
        case DType::F32: return "((float)" + c_float_str(f) + ")";
        case DType::F16: return "((_Float16)" + c_float_str(f) + ")";
        case DType::F64: return c_float_str(f);
        case DType::I8: case DType::I16: case DType::I32:
            snprintf(buf, sizeof buf, "((%s)(%" PRId64 "))", dtype_c_name(dtype), i);
            return buf;
        case DType::I64:
            if (i == std::numeric_limits<int64_t>::min()) return "((int64_t)(-9223372036854775807ll - 1))";
            snprintf(buf, sizeof buf, "((int64_t)(%" PRId64 "ll))", i);
            return buf;
        case DType::U8: case DType::U16: case DType::U32:
            snprintf(buf, sizeof buf, "((%s)(%" PRIu64 "u))", dtype_c_name(dtype), u);
            return buf;
        case DType::U64:
            snprintf(buf, sizeof buf, "((uint64_t)(%" PRIu64 "ull))", u);
            return buf;
        case DType::Bool: return u ? "true" : "false";
    }
    fail("invalid dtype");
}

std::string DScalar::to_string() const {
    char buf[64];
    if (is_float()) snprintf(buf, sizeof buf, "%g", f);
    else if (is_signed_int()) snprintf(buf, sizeof buf, "%" PRId64, i);
    else if (dtype == DType::Bool) snprintf(buf, sizeof buf, "%s", u ? "true" : "false");
    else snprintf(buf, sizeof buf, "%" PRIu64, u);
    return std::string(buf) + dtype_name(dtype);
}

Specials dtype_specials(DType t) {
    Specials s;
    const double inf = std::numeric_limits<double>::infinity();
    switch (t) {
        case DType::F32: s = {DScalar::f32(0), DScalar::f32(1), DScalar::f32((float) -inf), DScalar::f32((float) inf)}; break;
        case DType::F64: s = {DScalar::f64(0), DScalar::f64(1), DScalar::f64(-inf), DScalar::f64(inf)}; break;
        case DType::F16: s = {DScalar::f16(0), DScalar::f16(1), DScalar::f16((float) -inf), DScalar::f16((float) inf)}; break;
        case DType::I8: s = {DScalar::sint(t, 0), DScalar::sint(t, 1), DScalar::sint(t, INT8_MIN), DScalar::sint(t, INT8_MAX)}; break;
        case DType::I16: s = {DScalar::sint(t, 0), DScalar::sint(t, 1), DScalar::sint(t, INT16_MIN), DScalar::sint(t, INT16_MAX)}; break;
        case DType::I32: s = {DScalar::sint(t, 0), DScalar::sint(t, 1), DScalar::sint(t, INT32_MIN), DScalar::sint(t, INT32_MAX)}; break;
        case DType::I64: s = {DScalar::sint(t, 0), DScalar::sint(t, 1), DScalar::sint(t, INT64_MIN), DScalar::sint(t, INT64_MAX)}; break;
        case DType::U8: s = {DScalar::uint(t, 0), DScalar::uint(t, 1), DScalar::uint(t, 0), DScalar::uint(t, UINT8_MAX)}; break;
        case DType::U16: s = {DScalar::uint(t, 0), DScalar::uint(t, 1), DScalar::uint(t, 0), DScalar::uint(t, UINT16_MAX)}; break;
        case DType::U32: s = {DScalar::uint(t, 0), DScalar::uint(t, 1), DScalar::uint(t, 0), DScalar::uint(t, UINT32_MAX)}; break;
        case DType::U64: s = {DScalar::uint(t, 0), DScalar::uint(t, 1), DScalar::uint(t, 0), DScalar::uint(t, UINT64_MAX)}; break;
        case DType::Bool: s = {DScalar::boolean(false), DScalar::boolean(true), DScalar::boolean(false), DScalar::boolean(true)}; break;
    }
    return s;
}

HostTensor::HostTensor(DType dtype_, std::vector<size_t> shape_) : dtype(dtype_), shape(std::move(shape_)) {
    data = std::make_shared<std::vector<uint8_t>>(nbytes(), 0);
}

HostTensor::HostTensor(DType dtype_, std::vector<size_t> shape_, const void *src) : dtype(dtype_), shape(std::move(shape_)) {
    size_t n = nbytes();
    data = std::make_shared<std::vector<uint8_t>>(n);
    if (n) std::memcpy(data->data(), src, n);
    if (dtype == DType::Bool) {
        for (auto &b : *data) KN_ASSERT(b <= 1, "bool tensors must hold 0 or 1");
    }
}

HostTensor HostTensor::reshape(std::vector<size_t> new_shape) const {
    HostTensor r;
    r.dtype = dtype;
    r.shape = std::move(new_shape);
    r.data = data;
    KN_ASSERT(r.len() == len(), "reshape must keep the element count");
    return r;
}

bool HostTensor::equals(const HostTensor &o) const {
    if (dtype != o.dtype || shape != o.shape) return false;
    if (data == o.data) return true;
    if (!dtype_is_float(dtype)) return std::memcmp(bytes(), o.bytes(), nbytes()) == 0;
    size_t n = len();
    for (size_t k = 0; k < n; k++)
        if (at(k) != o.at(k)) return false;
    return true;
}

uint64_t HostTensor::hash() const {
    uint64_t h = (uint64_t) dtype;
    for (size_t d : shape) h = hash_combine(h, d);
    size_t n = std::min<size_t>(len(), 8);
    for (size_t k = 0; k < n; k++) {
        DScalar s = at(k);
        uint64_t bits;
        if (s.is_float()) {
            double v = std::isnan(s.f) ? std::numeric_limits<double>::quiet_NaN() : (s.f == 0 ? 0.0 : s.f);
            std::memcpy(&bits, &v, 8);
        } else {
            bits = s.u;
        }
        h = hash_combine(h, bits);
    }
    return h;
}

HostTensor HostTensor::scalar(const DScalar &s) {
    HostTensor t(s.dtype, {});
    t.set(0, s);
    return t;
}

}  // namespace kn
