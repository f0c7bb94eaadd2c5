#include "kernels.h"

#include <cinttypes>
#include <cstdlib>
#include <functional>

namespace kn {

namespace {
thread_local const GeneratorOptions *g_generator_options = nullptr;
const GeneratorOptions g_default_generator_options{};
}  // namespace

GeneratorScope::GeneratorScope(const GeneratorOptions &options) : previous_(g_generator_options), mine_(options) {
    g_generator_options = &mine_;
}
GeneratorScope::~GeneratorScope() { g_generator_options = previous_; }
const GeneratorOptions &generator_options() { return g_generator_options ? *g_generator_options : g_default_generator_options; }


// ------------------------------------------------------------------------------------------------ prelude

const char *kernel_prelude() {
    return R"KN(
typedef signed char kn_i8; typedef short kn_i16; typedef int kn_i32; typedef long long kn_i64;
typedef unsigned char kn_u8; typedef unsigned short kn_u16; typedef unsigned int kn_u32; typedef unsigned long long kn_u64;
#define int8_t kn_i8
#define int16_t kn_i16
#define int32_t kn_i32
#define int64_t kn_i64
#define uint8_t kn_u8
#define uint16_t kn_u16
#define uint32_t kn_u32
#define uint64_t kn_u64
#define KN_DEV __device__ __forceinline__
#define KN_INF (__builtin_inff())

template<typename T, typename U> KN_DEV T kn_bit_cast(U v) {
    static_assert(sizeof(T) == sizeof(U), "bit cast needs equal sizes");
    T r; __builtin_memcpy(&r, &v, sizeof(T)); return r;
}

// round an f32 value to the nearest f16 value (ties to even) and back
KN_DEV float kn_r16(float x) { return (float) (_Float16) x; }

// Abramowitz-Stegun erf, evaluated in f64 exactly like the host reference does
KN_DEV double kn_erf(double x) {
    double s = (x != x) ? x : (__builtin_signbit(x) ? -1.0 : 1.0);
    // (from 10 on the result is 1 to the last bit of an f64; the sixteenth power stays finite for the reciprocal below)
    double a = __builtin_fmin(__builtin_fabs(x), 10.0);
    double d = 1.0, p = a;
    d += 0.0705230784 * p; p *= a;
    d += 0.0422820123 * p; p *= a;
    d += 0.0092705272 * p; p *= a;
    d += 0.0001520143 * p; p *= a;
    d += 0.0002765672 * p; p *= a;
    d += 0.0000430638 * p;
    double d2 = d * d, d4 = d2 * d2, d8 = d4 * d4, d16 = d8 * d8;
    // 1 / d16 from the hardware's approximation and two Newton steps (d16 is finite and at least 1) instead of a
    // division with its scaling and fix-up, which was most of the function: 64M halves 99 -> 89 us, GELU over 64M floats 100 -> 89 us
    double r = __builtin_amdgcn_rcp(d16);
    r = __builtin_fma(__builtin_fma(-d16, r, 1.0), r, r);
    r = __builtin_fma(__builtin_fma(-d16, r, 1.0), r, r);
    return s * (1.0 - r);
}

// x * tanh(log(1 + e^x)) with tanh(log(u)) = (u^2 - 1) / (u^2 + 1) written out: n = e^x (e^x + 2), n / (n + 2). One
// exponential and one division instead of three library calls (64M floats: 219 -> 85 us, 64M halves 229 -> 60 us); no cancellation anywhere
// (for very negative x it is x e^x to rounding); from 20 on the factor is 1 in f32 and e^2x would overflow later.
KN_DEV float kn_mish(float x) {
    const float w = expf(x), n = w * (w + 2.0f);
    return x > 20.0f ? x : x * (n / (n + 2.0f));
}

// log(1 + w) for 0 <= w <= 1 as log(u) * w / (u - 1) with u = 1 + w rounded (u - 1 is exact, and the quotient puts
// back what the rounding of u took away); w itself where 1 + w rounds to 1. The library's log1pf costs several times
// an exponential (softplus over 64M floats: 198 -> 86 us, what the memory takes).
KN_DEV float kn_log1p_unit(float w) {
    const float u = 1.0f + w;
    return u == 1.0f ? w : logf(u) * (w / (u - 1.0f));
}

// The same three functions for halves. A result that is rounded to 11 bits does not need the library's exponential and
// logarithm (about twenty instructions each, which rows of halves then wait for instead of memory): the hardware's 2^x
// and log2 are a few 1e-7 off. The error function keeps the reference's polynomial (kn-graph/src/graph.rs:1677-1690)
// but in f32, written without the cancellation of 1 - 1 / d^16: with d = 1 + t, d^16 - 1 comes from squaring
// (1 + t)^2 - 1 = t (2 + t) four times, all terms positive, and erf = (d^16 - 1) / d^16.
KN_DEV float kn_mish_half(float x) {
    const float w = __expf(x), n = w * (w + 2.0f);
    return x > 20.0f ? x : x * (n * __frcp_rn(n + 2.0f));
}
KN_DEV float kn_erf_half(float x) {
    if (x != x) return x;
    const float a = fminf(__builtin_fabsf(x), 4.5f);
    float t = a * (0.0705230784f + a * (0.0422820123f + a * (0.0092705272f + a * (0.0001520143f + a * (0.0002765672f + a * 0.0000430638f)))));
    t = t * (2.0f + t);
    t = t * (2.0f + t);
    t = t * (2.0f + t);
    t = t * (2.0f + t);
    return __builtin_copysignf(t * __frcp_rn(1.0f + t), x);
}

// low 64 bits of the value converted to a 128 bit signed integer: truncation toward zero, saturation at the
// 128 bit bounds, NaN gives 0. Narrower integer targets wrap from here.
KN_DEV kn_u64 kn_f2i(double x) {
    kn_u64 bits = kn_bit_cast<kn_u64>(x);
    bool neg = (bits >> 63) != 0;
    int exp = (int) ((bits >> 52) & 0x7ff);
    kn_u64 mant = bits & 0xfffffffffffffull;
    if (exp == 0x7ff) return (mant != 0) ? 0ull : (neg ? 0ull : ~0ull);
    if (exp == 0) return 0ull;
    mant |= 1ull << 52;
    int e = exp - 1075;
    kn_u64 low;
    if (e >= 0) {
        if (exp - 1023 >= 127) return neg ? 0ull : ~0ull;
        low = e >= 64 ? 0ull : (mant << e);
    } else {
        low = (-e) >= 64 ? 0ull : (mant >> (-e));
    }
    return neg ? (0ull - low) : low;
}

template<typename T> KN_DEV T kn_shfl_xor(T v, int mask) {
    if constexpr (sizeof(T) <= 4) {
        int w = 0; __builtin_memcpy(&w, &v, sizeof(T));
        w = __shfl_xor(w, mask, 64);
        __builtin_memcpy(&v, &w, sizeof(T));
        return v;
    } else {
        static_assert(sizeof(T) % 4 == 0, "shuffled word by word");
        int w[sizeof(T) / 4]; __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
        for (unsigned i = 0; i < sizeof(T) / 4; i++) w[i] = __shfl_xor(w[i], mask, 64);
        __builtin_memcpy(&v, w, sizeof(T));
        return v;
    }
}

// butterfly reduction over aligned groups of G consecutive lanes (G a power of two, at most 64); every lane of
// the group ends up with the result
template<int G, typename T, typename F> KN_DEV T kn_group_reduce(T v, F f) {
#pragma unroll
    for (int m = G / 2; m > 0; m >>= 1) v = f(v, kn_shfl_xor(v, m));
    return v;
}

// reduction over a whole workgroup of NW waves through LDS; every thread gets the result. Each call site owns
// its `lds` slots and uses them once, so a single barrier between the partial writes and the reads is enough.
template<int NW, typename T, typename F> KN_DEV T kn_block_reduce(T v, F f, T *lds) {
    v = kn_group_reduce<64>(v, f);
    if constexpr (NW > 1) {
        if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
        __syncthreads();
        v = lds[0];
#pragma unroll
        for (int w = 1; w < NW; w++) v = f(v, lds[w]);
    }
    return v;
}

// Mean and centred sum of squares of a row out of per-lane statistics over `cnt` elements each, combined pairwise
// (Chan, Golub, LeVeque: M2 = M2a + M2b + (mean_b - mean_a)^2 * n / 2 for equal counts; no cancellation), in ONE
// pass over the G lanes of a group. Both partners of an exchange compute bit-identical results.
template<int G> KN_DEV void kn_group_stats(float &mean, float &m2, float cnt) {
#pragma unroll
    for (int m = 1; m < G; m <<= 1) {
        const float om = kn_shfl_xor(mean, m), o2 = kn_shfl_xor(m2, m);
        const float d = om - mean;
        m2 = (m2 + o2) + d * d * (cnt * 0.5f);
        mean = (mean + om) * 0.5f;
        cnt *= 2.0f;
    }
}

// the same over a workgroup of NW waves (a power of two), with one barrier; `lds` holds 2 * NW floats
template<int NW> KN_DEV void kn_block_stats(float &mean, float &m2, float cnt, float *lds) {
    kn_group_stats<64>(mean, m2, cnt);
    if constexpr (NW > 1) {
        cnt *= 64.0f;
        if ((threadIdx.x & 63) == 0) {
            lds[2 * (threadIdx.x >> 6)] = mean;
            lds[2 * (threadIdx.x >> 6) + 1] = m2;
        }
        __syncthreads();
        float ms[NW], qs[NW];
#pragma unroll
        for (int w = 0; w < NW; w++) {
            ms[w] = lds[2 * w];
            qs[w] = lds[2 * w + 1];
        }
#pragma unroll
        for (int n = NW; n > 1; n >>= 1) {
#pragma unroll
            for (int i = 0; i < n / 2; i++) {
                const float d = ms[2 * i + 1] - ms[2 * i];
                qs[i] = (qs[2 * i] + qs[2 * i + 1]) + d * d * (cnt * 0.5f);
                ms[i] = (ms[2 * i] + ms[2 * i + 1]) * 0.5f;
            }
            cnt *= 2.0f;
        }
        mean = ms[0];
        m2 = qs[0];
    }
}
)KN";
}

// ------------------------------------------------------------------------------------------------ small helpers

namespace {

// the type a value of this dtype has while it sits in registers
const char *compute_type(DType t) {
    switch (t) {
        case DType::F16: return "float";
        case DType::Bool: return "bool";
        default: return dtype_c_name(t);
    }
}

// the type used for loads and stores
const char *storage_type(DType t) {
    switch (t) {
        case DType::Bool: return "uint8_t";
        default: return dtype_c_name(t);
    }
}

std::string from_storage(DType t, const std::string &e) {
    if (t == DType::Bool) return "((" + e + ") != 0)";
    if (t == DType::F16) return "((float) (" + e + "))";
    return e;
}

std::string to_storage(DType t, const std::string &e) {
    if (t == DType::Bool) return "((uint8_t) ((" + e + ") ? 1 : 0))";
    if (t == DType::F16) return "((_Float16) (" + e + "))";
    return e;
}

std::string i64_str(int64_t v) {
    char buf[32];
    snprintf(buf, sizeof buf, "%" PRId64, v);
    return buf;
}

std::string int_array(const std::vector<int64_t> &v) {
    std::string r = "{";
    for (size_t i = 0; i < v.size(); i++) {
        if (i) r += ", ";
        r += i64_str(v[i]);
    }
    if (v.empty()) r += "0";
    return r + "}";
}

std::string fn(bool is_f64, const char *name) { return is_f64 ? std::string(name) : std::string(name) + "f"; }

std::string unary_expr(const ScalarNode &n, DType in, const std::string &x) {
    bool d = in == DType::F64;
    switch (n.unary) {
        case UnaryOp::Abs:
            if (dtype_is_float(in)) return fn(d, "__builtin_fabs") + "(" + x + ")";
            // wrapping two's complement abs
            return std::string("((") + dtype_c_name(in) + ") ((" + x + ") < 0 ? (0 - (uint64_t) (" + x + ")) : (uint64_t) (" + x + ")))";
        case UnaryOp::Neg:
            if (dtype_is_float(in)) return "(-(" + x + "))";
            return std::string("((") + dtype_c_name(in) + ") (0 - (uint64_t) (" + x + ")))";
        case UnaryOp::Sin: return fn(d, "sin") + "(" + x + ")";
        case UnaryOp::Cos: return fn(d, "cos") + "(" + x + ")";
        case UnaryOp::Exp: return fn(d, "exp") + "(" + x + ")";
        case UnaryOp::Log: return fn(d, "log") + "(" + x + ")";
        case UnaryOp::Sqrt: return fn(d, "sqrt") + "(" + x + ")";
        case UnaryOp::Sigmoid:
            // (halves: the hardware's 2^x and reciprocal, a few 1e-6 off before the result is rounded to 11 bits;
            // 64M halves 54.9 -> 43.8 us)
            if (in == DType::F16) return "__frcp_rn(1.0f + __expf(-(" + x + ")))";
            return d ? "(1.0 / (1.0 + exp(-(" + x + "))))" : "(1.0f / (1.0f + expf(-(" + x + "))))";
        case UnaryOp::Tanh: return fn(d, "tanh") + "(" + x + ")";
        case UnaryOp::Erf:
            if (in == DType::F16) return "kn_erf_half(" + x + ")";
            return d ? "kn_erf(" + x + ")" : "((float) kn_erf((double) (" + x + ")))";
        case UnaryOp::Mish:
            if (in == DType::F16) return "kn_mish_half(" + x + ")";
            if (!d) return "kn_mish(" + x + ")";
            return "((" + x + ") * " + fn(d, "tanh") + "(" + fn(d, "log1p") + "(" + fn(d, "exp") + "(" + x + "))))";
        case UnaryOp::Softplus:
            // (halves: 1 + e^-|x| rounded to f32 is off by at most 6e-8, half a unit of the last place of the smallest
            // normal half; the hardware's 2^x and log2)
            if (in == DType::F16) return "(__logf(1.0f + __expf(-__builtin_fabsf(" + x + "))) + fmaxf(" + x + ", 0.0f))";
            if (!d) return "(kn_log1p_unit(expf(-__builtin_fabsf(" + x + "))) + fmaxf(" + x + ", 0.0f))";
            return "(" + fn(d, "log1p") + "(" + fn(d, "exp") + "(-" + fn(d, "__builtin_fabs") + "(" + x + "))) + " + fn(d, "fmax") + "(" + x + ", " + (d ? "0.0" : "0.0f") + "))";
        case UnaryOp::ValueCast: {
            DType to = n.cast_to;
            if (to == DType::Bool) return "((" + x + ") != 0)";
            if (in == DType::Bool) return std::string("((") + compute_type(to) + ") ((" + x + ") ? 1 : 0))";
            if (dtype_is_float(in)) {
                if (dtype_is_float(to)) return std::string("((") + compute_type(to) + ") (" + x + "))";
                return std::string("((") + dtype_c_name(to) + ") kn_f2i((double) (" + x + ")))";
            }
            // integer source: floats go through f64 first, integers wrap
            if (to == DType::F64) return "((double) (" + x + "))";
            if (dtype_is_float(to)) return "((float) (double) (" + x + "))";
            return std::string("((") + dtype_c_name(to) + ") (" + x + "))";
        }
        case UnaryOp::BitCast: {
            // f16 values live in registers as float: go through the storage type
            std::string src = in == DType::F16 ? "((_Float16) (" + x + "))" : x;
            std::string r = std::string("kn_bit_cast<") + storage_type(n.cast_to) + ">(" + src + ")";
            return n.cast_to == DType::F16 ? "((float) " + r + ")" : r;
        }
    }
    fail("invalid unary op");
}

std::string binary_expr(BinaryOp op, DType t, const std::string &a, const std::string &b) {
    if (t == DType::Bool) {
        switch (op) {
            case BinaryOp::Add: case BinaryOp::Max: return "((" + a + ") || (" + b + "))";
            case BinaryOp::Mul: case BinaryOp::Min: return "((" + a + ") && (" + b + "))";
            case BinaryOp::Sub: case BinaryOp::Div: return "((" + a + ") && !(" + b + "))";
            default: fail("unsupported bool operation");
        }
    }
    bool fl = dtype_is_float(t), d = t == DType::F64;
    std::string T = dtype_c_name(t);
    switch (op) {
        case BinaryOp::Add: case BinaryOp::Sub: case BinaryOp::Mul: {
            const char *sym = op == BinaryOp::Add ? "+" : op == BinaryOp::Sub ? "-" : "*";
            if (fl) return "((" + a + ") " + sym + " (" + b + "))";
            // wrap in unsigned arithmetic so that signed overflow is defined
            return "((" + T + ") ((uint64_t) (" + a + ") " + sym + " (uint64_t) (" + b + ")))";
        }
        case BinaryOp::Div:
            if (fl) return "((" + a + ") / (" + b + "))";
            if (dtype_is_signed(t)) return "((" + b + ") == -1 ? (" + T + ") (0 - (uint64_t) (" + a + ")) : (" + T + ") ((" + a + ") / (" + b + ")))";
            return "((" + T + ") ((" + a + ") / (" + b + ")))";
        case BinaryOp::Min:
            if (fl) return fn(d, "fmin") + "(" + a + ", " + b + ")";
            return "((" + a + ") < (" + b + ") ? (" + a + ") : (" + b + "))";
        case BinaryOp::Max:
            if (fl) return fn(d, "fmax") + "(" + a + ", " + b + ")";
            return "((" + a + ") > (" + b + ") ? (" + a + ") : (" + b + "))";
        case BinaryOp::Pow:
            if (!fl) fail("Pow is only supported for floats");
            return fn(d, "pow") + "(" + a + ", " + b + ")";
    }
    fail("invalid binary op");
}

// Emit the statements of an expression. `load` names the already loaded register value for an operand.
// Returns the name of the result variable.
template <typename LoadName>
std::string emit_expr(std::ostringstream &ss, const ScalarExpr &expr, const std::string &prefix, LoadName load,
                      const char *indent = "    ") {
    KN_ASSERT(!expr.nodes.empty());
    for (size_t i = 0; i < expr.nodes.size(); i++) {
        const ScalarNode &n = expr.nodes[i];
        std::string name = prefix + std::to_string(i);
        std::string rhs;
        switch (n.kind) {
            case ScalarNode::Load: rhs = load(n.operand); break;
            case ScalarNode::Const: rhs = n.constant.to_c_str(); break;
            case ScalarNode::Unary: rhs = unary_expr(n, expr.nodes[n.a].dtype, prefix + std::to_string(n.a)); break;
            case ScalarNode::Binary: {
                const ScalarNode &rn = expr.nodes[n.b];
                // a square, a cube or a square root written as a power (what `x ** 2` of a mean of squares arrives as):
                // the library call is about a hundred instructions (64M floats: 252 us against 86 us for the product)
                const bool const_power = n.binary == BinaryOp::Pow && rn.kind == ScalarNode::Const && dtype_is_float(rn.constant.dtype);
                const std::string base = prefix + std::to_string(n.a);
                if (const_power && rn.constant.f == 2.0)
                    rhs = "((" + base + ") * (" + base + "))";
                else if (const_power && rn.constant.f == 3.0)
                    rhs = "((" + base + ") * (" + base + ") * (" + base + "))";
                else if (const_power && rn.constant.f == 1.5 && rn.constant.dtype != DType::F64)
                    // x sqrt(x): NaN below zero like the power, +0 for -0 (the product of two -0); only -inf needs a word
                    // (64M floats: 238 -> what the memory takes)
                    rhs = "((" + base + ") == -KN_INF ? KN_INF : ((" + base + ") * sqrtf(" + base + ")))";
                else if (const_power && rn.constant.f == 0.5 && rn.constant.dtype != DType::F64)
                    // (pow(-0, 0.5) is +0 and pow(-inf, 0.5) is +inf, where the square root gives -0 and NaN)
                    rhs = "((" + base + ") == -KN_INF ? KN_INF : (sqrtf(" + base + ") + 0.0f))";
                else
                    rhs = binary_expr(n.binary, expr.nodes[n.a].dtype, prefix + std::to_string(n.a), prefix + std::to_string(n.b));
                break;
            }
            case ScalarNode::Raw: {
                // the caller's statements in a block of their own, with x0 pointing at the result and xk at loaded operand k
                KN_ASSERT(i + 1 == expr.nodes.size(), "a raw operation is the last node of its expression");
                ss << indent << compute_type(n.dtype) << " " << name << "_v = " << compute_type(n.dtype) << "();\n" << indent << "{\n";
                ss << indent << "    " << compute_type(n.dtype) << " *const x0 = &" << name << "_v;\n";
                for (size_t j = 0; j < i; j++) {
                    const ScalarNode &in = expr.nodes[j];
                    if (in.kind != ScalarNode::Load) continue;
                    ss << indent << "    const " << compute_type(in.dtype) << " *const x" << in.operand << " = &" << prefix << j << ";\n";
                    ss << indent << "    (void) x" << in.operand << ";\n";
                }
                ss << indent << "    " << n.raw << "\n" << indent << "}\n";
                rhs = name + "_v";
                break;
            }
        }
        // values of type f16 are kept as floats that are exactly representable in f16
        if (n.dtype == DType::F16 && (n.kind == ScalarNode::Unary || n.kind == ScalarNode::Binary || n.kind == ScalarNode::Raw)) rhs = "kn_r16(" + rhs + ")";
        ss << indent << "const " << compute_type(n.dtype) << " " << name << " = " << rhs << ";\n";
    }
    return prefix + std::to_string(expr.result());
}

// Axis bookkeeping shared by all kernels: drop unit axes, optionally order by the first operand's strides and
// merge neighbours that are contiguous for every operand.
struct Collapsed {
    std::vector<size_t> shape;
    std::vector<std::vector<int64_t>> strides;  // [operand][axis]
    size_t rank() const { return shape.size(); }
    size_t size() const { return concrete_size(shape); }
};

Collapsed collapse_axes(const std::vector<size_t> &shape, const std::vector<std::vector<int64_t>> &strides, bool reorder) {
    size_t n_ops = strides.size();
    std::vector<size_t> axes;
    for (size_t a = 0; a < shape.size(); a++)
        if (shape[a] != 1) axes.push_back(a);
    if (reorder) {
        std::stable_sort(axes.begin(), axes.end(),
                         [&](size_t x, size_t y) { return std::llabs(strides[0][x]) > std::llabs(strides[0][y]); });
    }
    Collapsed c;
    c.strides.resize(n_ops);
    for (size_t a : axes) {
        bool merged = false;
        if (!c.shape.empty()) {
            merged = true;
            for (size_t k = 0; k < n_ops; k++)
                merged &= c.strides[k].back() == strides[k][a] * (int64_t) shape[a];
            if (merged) {
                c.shape.back() *= shape[a];
                for (size_t k = 0; k < n_ops; k++) c.strides[k].back() = strides[k][a];
            }
        }
        if (!merged) {
            c.shape.push_back(shape[a]);
            for (size_t k = 0; k < n_ops; k++) c.strides[k].push_back(strides[k][a]);
        }
    }
    return c;
}

bool fits_i32(const std::vector<KernelOperand> &ops, size_t total) {
    if (total >= (1ull << 31)) return false;
    for (auto &op : ops) {
        auto [lo, hi] = op.shape.offset_bounds();
        if (lo <= -(1ll << 31) || hi >= (1ll << 31)) return false;
    }
    return true;
}

// Emit code that splits `var` (a flat index over `dims`, last axis fastest) into per-operand offsets.
// `offs[k]` are the names of the accumulators, which must already be declared.
void emit_decompose(std::ostringstream &ss, const std::string &indent, const std::string &var,
                    const std::vector<size_t> &dims, const std::vector<std::vector<int64_t>> &strides,
                    const std::vector<std::string> &offs) {
    size_t rank = dims.size();
    if (rank == 0) return;
    ss << indent << "{ idx_t kn_left = " << var << ";\n";
    for (size_t a = rank; a-- > 0;) {
        std::string c = "kn_c" + std::to_string(a);
        if (a == 0) ss << indent << "  const idx_t " << c << " = kn_left;\n";
        else {
            ss << indent << "  const idx_t " << c << " = kn_left % (idx_t) " << dims[a] << "; kn_left /= (idx_t) " << dims[a] << ";\n";
        }
        for (size_t k = 0; k < offs.size(); k++)
            if (strides[k][a] != 0) ss << indent << "  " << offs[k] << " += " << c << " * (idx_t) " << strides[k][a] << ";\n";
    }
    ss << indent << "}\n";
}

// Streaming heuristics: a big tensor that is touched exactly once per element gains nothing from the caches, and
// its dirty lines would only delay whatever runs next. Such operands are read and written with non-temporal
// accesses (GeneratorOptions::streaming_bytes).
size_t nt_threshold_bytes() {
    const size_t v = generator_options().streaming_bytes;
    return v == 0 ? SIZE_MAX : v;
}

bool is_streaming(const KernelOperand &op) {
    if (op.shape.size() * dtype_bytes(op.dtype) < nt_threshold_bytes()) return false;
    for (size_t a = 0; a < op.shape.rank(); a++)
        if (op.shape.shape()[a] > 1 && op.shape.strides()[a] == 0) return false;
    return true;
}

std::string load_expr(const std::string &type, const std::string &ptr, bool nt) {
    if (nt) return "__builtin_nontemporal_load((const " + type + " *) (" + ptr + "))";
    return "*(const " + type + " *) (" + ptr + ")";
}

std::string store_stmt(const std::string &type, const std::string &ptr, const std::string &value, bool nt) {
    if (nt) return "__builtin_nontemporal_store(" + value + ", (" + type + " *) (" + ptr + "));";
    return "*(" + type + " *) (" + ptr + ") = " + value + ";";
}

uint32_t ceil_div_u32(size_t a, size_t b) {
    size_t r = (a + b - 1) / b;
    if (r > 0x7fffffffull) fail("kernel grid too large: ", r);
    return (uint32_t) r;
}

void emit_header(std::ostringstream &ss, bool idx64, size_t n_ptrs) {
    ss << kernel_prelude();
    ss << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
    ss << "struct KnPtrs { void *p[" << std::max<size_t>(n_ptrs, 1) << "]; };\n";
}

// `element_aligned`: the vector may start at any element (the hardware takes 128 bit accesses at any address; the type
// says so, so that the compiler does not assume 16 byte alignment)
std::string vec_type_decl(const std::string &name, DType t, size_t vec, bool element_aligned = false) {
    std::string decl = std::string("typedef ") + storage_type(t) + " " + name + " __attribute__((ext_vector_type(" + std::to_string(vec) + ")";
    if (element_aligned) decl += ", aligned(" + std::to_string(dtype_bytes(t)) + ")";
    return decl + "));\n";
}

// Largest power-of-two vector width (in elements) such that every operand can be accessed with aligned vectors
// along the last collapsed axis. `inner_strides[k]` must be 0 or 1 for a width above one.
size_t pick_vec(const std::vector<KernelOperand> &ops, const Collapsed &c, size_t inner_size) {
    if (c.rank() == 0) return 1;
    size_t max_bytes = 1;
    for (auto &op : ops) max_bytes = std::max(max_bytes, dtype_bytes(op.dtype));
    size_t vec = 16 / max_bytes;
    size_t last = c.rank() - 1;
    for (; vec > 1; vec /= 2) {
        bool ok = inner_size % vec == 0;
        for (size_t k = 0; k < ops.size() && ok; k++) {
            int64_t is = c.strides[k][last];
            if (is != 0 && is != 1) ok = false;
            size_t es = dtype_bytes(ops[k].dtype);
            if (is == 1) {
                ok &= ops[k].offset_bytes % (int64_t) (vec * es) == 0;
                for (size_t a = 0; a < last; a++) ok &= c.strides[k][a] % (int64_t) vec == 0;
            }
        }
        if (ok) break;
    }
    return vec;
}

}  // namespace

// ------------------------------------------------------------------------------------------------ scalar kernel

KernelSpec make_scalar_kernel(const std::vector<KernelOperand> &operands, const ScalarExpr &expr) {
    return make_scalar_kernel_multi(operands, {expr});
}

namespace {

// Elementwise kernels with a transposed operand. When an input is contiguous along another axis than the outputs
// (a permuted view: NCHW -> tokens, a [k, n] weight read as [n, k]), neither order of the plain kernel's index
// space gives both sides wide accesses: lanes that run along the outputs' rows read the input with a stride, 4 or
// 2 useful bytes per cache line touched. Here a workgroup owns a tile of 64 x 64 elements (input axis x output axis): it
// reads the transposed operands with lanes along THEIR contiguous axis into LDS, then computes and stores with
// lanes along the outputs' axis, taking those operands from LDS. Rows of the LDS tile are padded so that both
// directions are free of bank conflicts.
std::optional<KernelSpec> make_transposed_tile_kernel(const std::vector<KernelOperand> &operands, const std::vector<ScalarExpr> &exprs,
                                                      const Collapsed &c, size_t total) {
    const bool enabled = generator_options().tiled_transpose;
    const size_t n_out = exprs.size(), n_ops = operands.size(), rank = c.rank();
    if (!enabled || rank < 2 || total < (1u << 16)) return std::nullopt;
    const size_t last = rank - 1;
    for (size_t o = 0; o < n_out; o++)
        if (c.strides[o][last] != 1) return std::nullopt;
    // the transposed operands, and the axis they all are contiguous along
    std::vector<bool> transposed(n_ops, false);
    std::optional<size_t> axis;
    size_t lds_bytes = 0;
    for (size_t k = n_out; k < n_ops; k++) {
        const int64_t inner = c.strides[k][last];
        if (inner == 0 || inner == 1) continue;
        std::optional<size_t> mine;
        for (size_t a = 0; a < last; a++)
            if (c.strides[k][a] == 1) mine = a;
        if (!mine || (axis && *axis != *mine)) return std::nullopt;
        axis = mine;
        transposed[k] = true;
    }
    if (!axis || c.shape[*axis] < 16 || c.shape[last] < 16) return std::nullopt;
    const size_t A = *axis, dim_a = c.shape[A], dim_l = c.shape[last];
    // Elements of one byte (u8, i8, bool): a row of 64 of them is half a cache line per wave. When every operand is
    // of that size and everything sits on 4 byte boundaries, a thread moves 4 neighbouring elements as one word and
    // the tile is 128 x 128 (a transposition of 16384 x 16384 bytes: 190 -> 115 us, 2.8 -> 4.7 TB/s).
    bool words = dim_a % 4 == 0 && dim_l % 4 == 0;
    for (size_t k = 0; k < n_ops && words; k++) {
        words = dtype_bytes(operands[k].dtype) == 1 && operands[k].offset_bytes % 4 == 0;
        for (size_t a = 0; a < rank && words; a++) {
            const int64_t st = c.strides[k][a];
            const bool unit_ok = (a == last && !transposed[k]) || (a == A && transposed[k]);
            words = unit_ok ? st == 1 : st % 4 == 0;
        }
    }
    const size_t TILE = words ? 128 : 64;
    auto pitch_of = [&](DType t) { return TILE + std::max<size_t>(1, 4 / dtype_bytes(t)); };
    for (size_t k = n_out; k < n_ops; k++)
        if (transposed[k]) lds_bytes += TILE * pitch_of(operands[k].dtype) * dtype_bytes(operands[k].dtype);
    if (lds_bytes > 48 * 1024) return std::nullopt;
    const size_t tiles_a = (dim_a + TILE - 1) / TILE, tiles_l = (dim_l + TILE - 1) / TILE;
    std::vector<size_t> rest_dims;
    std::vector<std::vector<int64_t>> rest_strides(n_ops);
    size_t rest = 1;
    for (size_t a = 0; a < last; a++) {
        if (a == A) continue;
        rest_dims.push_back(c.shape[a]);
        rest *= c.shape[a];
        for (size_t k = 0; k < n_ops; k++) rest_strides[k].push_back(c.strides[k][a]);
    }
    const size_t blocks = rest * tiles_a * tiles_l;
    if (blocks > 0x7fffffffull) return std::nullopt;
    const bool idx64 = !fits_i32(operands, total + TILE * TILE);

    KernelSpec spec;
    spec.name = "kn_scalar";
    spec.n_ptrs = n_ops;
    spec.block = 256;
    std::ostringstream ss;
    emit_header(ss, idx64, n_ops);
    for (size_t k = 0; k < n_ops; k++) ss << "typedef " << storage_type(operands[k].dtype) << " S" << k << ";\n";
    for (size_t o = 0; o < n_out; o++) {
        ss << "KN_DEV " << compute_type(operands[o].dtype) << " kn_op" << o << "(";
        for (size_t k = n_out; k < n_ops; k++) ss << (k > n_out ? ", " : "") << compute_type(operands[k].dtype) << " x" << k;
        ss << ") {\n";
        std::string res = emit_expr(ss, exprs[o], "y", [&](size_t operand) {
            KN_ASSERT(operand >= n_out && operand < n_ops);
            return "x" + std::to_string(operand);
        });
        ss << "    return " << res << ";\n}\n";
    }
    ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_scalar(KnPtrs ptrs) {\n";
    for (size_t k = 0; k < n_ops; k++) {
        ss << "    S" << k << " *p" << k << " = (S" << k << " *) ptrs.p[" << k << "];\n";
        if (transposed[k] && !words) ss << "    __shared__ S" << k << " tile" << k << "[" << TILE << "][" << pitch_of(operands[k].dtype) << "];\n";
        // (rows of 32 words and one of padding; row l of the tile sits in row (l % 4) * 32 + l / 4, so that the four
        // rows a thread gathers a word from lie 32 rows apart and the threads of a wave read 33 words apart)
        if (transposed[k] && words) ss << "    __shared__ unsigned int tile" << k << "[128][33];\n";
    }
    // Which tile: the output axis fastest, then the operands' axis, then everything else. Consecutive workgroups then
    // write neighbouring pieces of the same 64 rows, and read tiles that lie 64 rows of the transposed operand
    // apart: when that distance is (nearly) a multiple of 1 MB, as with rows of 16 KB or more whose length is a
    // power of two, all workgroups in flight read through the same few memory channels. Those shapes walk the tiles
    // along diagonals instead, which moves both sides on by a tile's width per workgroup (f32 8192 x 8192: 135 ->
    // 103 us, f16 16384 x 16384: 298 -> 227 us); other shapes lose the order of their writes that way (f32
    // 32768 x 2048: 119 -> 153 us) and keep the straight order.
    bool diagonal = false;
    for (size_t k = n_out; k < n_ops && !diagonal; k++) {
        if (!transposed[k]) continue;
        const uint64_t apart = (uint64_t) std::llabs(c.strides[k][last]) * dtype_bytes(operands[k].dtype) * TILE;
        const uint64_t off = apart % (1u << 20);
        diagonal = tiles_a > 1 && tiles_l > 1 && (off <= (1u << 15) || off >= (1u << 20) - (1u << 15));
        break;
    }
    ss << "    idx_t blk = (idx_t) blockIdx.x;\n";
    ss << "    const idx_t tl = blk % (idx_t) " << tiles_l << "; blk /= (idx_t) " << tiles_l << ";\n";
    if (!diagonal)
        ss << "    const idx_t ta = blk % (idx_t) " << tiles_a << "; blk /= (idx_t) " << tiles_a << ";\n";
    else
        ss << "    const idx_t ta = (blk % (idx_t) " << tiles_a << " + tl) % (idx_t) " << tiles_a << "; blk /= (idx_t) " << tiles_a << ";\n";
    ss << "    const idx_t l0 = tl * " << TILE << ", a0 = ta * " << TILE << ";\n";
    for (size_t k = 0; k < n_ops; k++) ss << "    idx_t off" << k << " = 0;\n";
    {
        std::vector<std::string> offs;
        for (size_t k = 0; k < n_ops; k++) offs.push_back("off" + std::to_string(k));
        emit_decompose(ss, "    ", "blk", rest_dims, rest_strides, offs);
    }
    auto offset_of = [&](size_t k, const std::string &a, const std::string &l) {
        std::string text = "off" + std::to_string(k);
        if (c.strides[k][A] != 0) text += " + (a0 + " + a + ") * (idx_t) " + std::to_string(c.strides[k][A]);
        if (c.strides[k][last] != 0) text += " + (l0 + " + l + ") * (idx_t) " + std::to_string(c.strides[k][last]);
        return text;
    };
    if (words) {
        ss << "    const int cw = threadIdx.x & 31, rw = threadIdx.x >> 5;\n";
        // phase 1: a word of 4 elements along the transposed operands' contiguous axis per thread
        ss << "    if (a0 + 4 * cw < (idx_t) " << dim_a << ") {\n#pragma unroll\n        for (int i = 0; i < 16; i++) {\n";
        ss << "            const int l = rw + 8 * i;\n            if (l0 + l < (idx_t) " << dim_l << ") {\n";
        for (size_t k = n_out; k < n_ops; k++)
            if (transposed[k])
                ss << "                tile" << k << "[(l & 3) * 32 + (l >> 2)][cw] = *(const unsigned int *) (p" << k << " + " << offset_of(k, "4 * cw", "l") << ");\n";
        ss << "            }\n        }\n    }\n    __syncthreads();\n";
        // phase 2: a word of 4 elements along the outputs' contiguous axis per thread
        ss << "    if (l0 + 4 * cw < (idx_t) " << dim_l << ") {\n";
        bool straight = false;
        for (size_t k = n_out; k < n_ops; k++)
            if (!transposed[k]) {
                straight = true;
                ss << "        unsigned int g" << k << "[16];\n";
            }
        if (straight) {
            ss << "#pragma unroll\n        for (int i = 0; i < 16; i++) {\n            const int a = rw + 8 * i;\n";
            ss << "            if (a0 + a < (idx_t) " << dim_a << ") {\n";
            for (size_t k = n_out; k < n_ops; k++)
                if (!transposed[k]) ss << "                g" << k << "[i] = *(const unsigned int *) (p" << k << " + " << offset_of(k, "a", "4 * cw") << ");\n";
            ss << "            }\n        }\n";
        }
        ss << "#pragma unroll\n        for (int i = 0; i < 16; i++) {\n";
        ss << "            const int a = rw + 8 * i;\n            if (a0 + a < (idx_t) " << dim_a << ") {\n";
        for (size_t o = 0; o < n_out; o++) ss << "                unsigned int w" << o << " = 0;\n";
        ss << "#pragma unroll\n                for (int j = 0; j < 4; j++) {\n";
        for (size_t k = n_out; k < n_ops; k++) {
            ss << "                    const S" << k << " r" << k << " = (S" << k << ") ((";
            if (transposed[k]) ss << "tile" << k << "[j * 32 + cw][a >> 2] >> (8 * (a & 3))";
            else ss << "g" << k << "[i] >> (8 * j)";
            ss << ") & 0xffu);\n";
        }
        for (size_t o = 0; o < n_out; o++) {
            std::string call = "kn_op" + std::to_string(o) + "(";
            for (size_t k = n_out; k < n_ops; k++) call += (k > n_out ? ", " : "") + from_storage(operands[k].dtype, "r" + std::to_string(k));
            call += ")";
            ss << "                    w" << o << " |= (unsigned int) (uint8_t) " << to_storage(operands[o].dtype, call) << " << (8 * j);\n";
        }
        ss << "                }\n";
        for (size_t o = 0; o < n_out; o++) ss << "                *(unsigned int *) (p" << o << " + " << offset_of(o, "a", "4 * cw") << ") = w" << o << ";\n";
        ss << "            }\n        }\n    }\n}\n";
        spec.source = ss.str();
        spec.grid = (uint32_t) blocks;
        std::ostringstream note;
        note << "rank=" << rank << " transposed tiles 128x128 of bytes, a word per thread" << (diagonal ? ", along diagonals" : "") << " idx=" << (idx64 ? 64 : 32);
        if (n_out > 1) note << " outputs=" << n_out;
        spec.strategy = note.str();
        return spec;
    }
    ss << "    const int lane = threadIdx.x & 63, row = threadIdx.x >> 6;\n";
    // phase 1: lanes along the transposed operands' contiguous axis
    ss << "    if (a0 + lane < (idx_t) " << dim_a << ") {\n#pragma unroll\n        for (int i = 0; i < 16; i++) {\n";
    ss << "            const int l = row + 4 * i;\n            if (l0 + l < (idx_t) " << dim_l << ") {\n";
    for (size_t k = n_out; k < n_ops; k++)
        if (transposed[k]) ss << "                tile" << k << "[l][lane] = p" << k << "[" << offset_of(k, "lane", "l") << "];\n";
    ss << "            }\n        }\n    }\n    __syncthreads();\n";
    // phase 2: lanes along the outputs' contiguous axis. The operands that are read straight from global memory
    // are all requested before the first store (a load may not pass a store that might alias it).
    ss << "    if (l0 + lane < (idx_t) " << dim_l << ") {\n";
    bool any_straight = false;
    for (size_t k = n_out; k < n_ops; k++) {
        if (transposed[k]) continue;
        any_straight = true;
        ss << "        S" << k << " g" << k << "[16];\n";
    }
    if (any_straight) {
        ss << "#pragma unroll\n        for (int i = 0; i < 16; i++) {\n            const int a = row + 4 * i;\n";
        ss << "            if (a0 + a < (idx_t) " << dim_a << ") {\n";
        for (size_t k = n_out; k < n_ops; k++)
            if (!transposed[k]) ss << "                g" << k << "[i] = p" << k << "[" << offset_of(k, "a", "lane") << "];\n";
        ss << "            }\n        }\n";
    }
    ss << "#pragma unroll\n        for (int i = 0; i < 16; i++) {\n";
    ss << "            const int a = row + 4 * i;\n            if (a0 + a < (idx_t) " << dim_a << ") {\n";
    for (size_t k = n_out; k < n_ops; k++) {
        ss << "                const S" << k << " r" << k << " = ";
        if (transposed[k]) ss << "tile" << k << "[lane][a];\n";
        else ss << "g" << k << "[i];\n";
    }
    for (size_t o = 0; o < n_out; o++) {
        std::string call = "kn_op" + std::to_string(o) + "(";
        for (size_t k = n_out; k < n_ops; k++) call += (k > n_out ? ", " : "") + from_storage(operands[k].dtype, "r" + std::to_string(k));
        call += ")";
        ss << "                p" << o << "[" << offset_of(o, "a", "lane") << "] = " << to_storage(operands[o].dtype, call) << ";\n";
    }
    ss << "            }\n        }\n    }\n}\n";
    spec.source = ss.str();
    spec.grid = (uint32_t) blocks;
    std::ostringstream note;
    note << "rank=" << rank << " transposed tiles " << TILE << "x" << TILE << (diagonal ? " along diagonals" : "") << " idx=" << (idx64 ? 64 : 32);
    if (n_out > 1) note << " outputs=" << n_out;
    spec.strategy = note.str();
    return spec;
}

}  // namespace

KernelSpec make_scalar_kernel_multi(const std::vector<KernelOperand> &operands, const std::vector<ScalarExpr> &exprs) {
    const size_t n_out = exprs.size();
    KN_ASSERT(n_out >= 1 && operands.size() >= n_out);
    const std::vector<size_t> &shape = operands[0].shape.shape();
    std::vector<std::vector<int64_t>> strides;
    for (auto &op : operands) {
        KN_ASSERT(op.shape.shape() == shape, "all operands of an elementwise kernel must have the same shape");
        strides.push_back(op.shape.strides());
    }
    for (size_t o = 0; o < n_out; o++) KN_ASSERT(exprs[o].nodes.back().dtype == operands[o].dtype);

    KernelSpec spec;
    spec.name = "kn_scalar";
    spec.n_ptrs = operands.size();
    spec.block = 256;
    size_t total = concrete_size(shape);
    if (total == 0) return spec;

    Collapsed c = collapse_axes(shape, strides, true);
    if (c.rank() == 0) {
        c.shape = {1};
        for (auto &s : c.strides) s = {1};
    }
    size_t rank = c.rank();
    size_t inner = c.shape[rank - 1];
    size_t vec = pick_vec(operands, c, inner);
    if (vec == 1)
        if (auto tiled = make_transposed_tile_kernel(operands, exprs, c, total)) return *tiled;
    size_t total_vecs = total / vec;
    size_t unroll = total_vecs >= 256 * 4 * 1024 ? 4 : (total_vecs >= 256 * 2 * 512 ? 2 : 1);
    bool idx64 = !fits_i32(operands, total + 256 * unroll);

    std::ostringstream ss;
    emit_header(ss, idx64, operands.size());
    for (size_t k = 0; k < operands.size(); k++) {
        ss << "typedef " << storage_type(operands[k].dtype) << " S" << k << ";\n";
        if (vec > 1) ss << vec_type_decl("V" + std::to_string(k), operands[k].dtype, vec);
    }
    // the fused expressions, one per output; every one takes all loaded operands
    for (size_t o = 0; o < n_out; o++) {
        ss << "KN_DEV " << compute_type(operands[o].dtype) << " kn_op" << o << "(";
        for (size_t k = n_out; k < operands.size(); k++) ss << (k > n_out ? ", " : "") << compute_type(operands[k].dtype) << " x" << k;
        ss << ") {\n";
        std::string res = emit_expr(ss, exprs[o], "y", [&](size_t operand) {
            KN_ASSERT(operand >= n_out && operand < operands.size());
            return "x" + std::to_string(operand);
        });
        ss << "    return " << res << ";\n}\n";
    }

    // dims in vector units along the last axis
    std::vector<size_t> dims = c.shape;
    dims[rank - 1] = inner / vec;
    std::vector<std::vector<int64_t>> vstrides = c.strides;
    for (auto &s : vstrides) s[rank - 1] *= (int64_t) vec;

    ss << "#define UNROLL " << unroll << "\n#define VEC " << vec << "\n";
    ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_scalar(KnPtrs ptrs) {\n";
    for (size_t k = 0; k < operands.size(); k++) ss << "    S" << k << " *p" << k << " = (S" << k << " *) ptrs.p[" << k << "];\n";
    ss << "    const idx_t total = (idx_t) " << total_vecs << ";\n";
    ss << "    const idx_t base = (idx_t) blockIdx.x * (idx_t) (256 * UNROLL) + (idx_t) threadIdx.x;\n";
    ss << "    idx_t off[UNROLL][" << operands.size() << "];\n    bool ok[UNROLL];\n";
    for (size_t k = n_out; k < operands.size(); k++) {
        bool vload = vec > 1 && c.strides[k][rank - 1] == 1;
        ss << "    " << (vload ? "V" : "S") << k << " r" << k << "[UNROLL];\n";
    }
    // phase 1: addresses and loads, all issued before any arithmetic
    ss << "#pragma unroll\n    for (int u = 0; u < UNROLL; u++) {\n";
    // Vectors past the end are clamped for addressing and only their stores are masked, so that the loads are
    // straight-line code that the compiler issues back to back (a branch per load makes every load wait for the one
    // before it); a grid that covers the tensor exactly needs no check at all.
    const bool exact = total_vecs % (256 * unroll) == 0;
    if (exact) ss << "        const idx_t v = base + (idx_t) (u * 256);\n        ok[u] = true;\n";
    else ss << "        const idx_t v_raw = base + (idx_t) (u * 256);\n        ok[u] = v_raw < total;\n        const idx_t v = ok[u] ? v_raw : total - 1;\n";
    ss << "        for (int k = 0; k < " << operands.size() << "; k++) off[u][k] = 0;\n";
    ss << "        {\n";
    {
        std::vector<std::string> offs;
        for (size_t k = 0; k < operands.size(); k++) offs.push_back("off[u][" + std::to_string(k) + "]");
        emit_decompose(ss, "            ", "v", dims, vstrides, offs);
    }
    for (size_t k = n_out; k < operands.size(); k++) {
        bool vload = vec > 1 && c.strides[k][rank - 1] == 1;
        if (vload)
            ss << "            r" << k << "[u] = "
               << load_expr("V" + std::to_string(k), "p" + std::to_string(k) + " + off[u][" + std::to_string(k) + "]", is_streaming(operands[k])) << ";\n";
        else ss << "            r" << k << "[u] = p" << k << "[off[u][" << k << "]];\n";
    }
    ss << "        }\n    }\n";
    // phase 2: arithmetic and stores
    ss << "#pragma unroll\n    for (int u = 0; u < UNROLL; u++) {\n        if (ok[u]) {\n";
    for (size_t o = 0; o < n_out; o++) {
        const std::string os_name = std::to_string(o);
        auto call = [&](const std::string &j) {
            std::string text = "kn_op" + os_name + "(";
            for (size_t k = n_out; k < operands.size(); k++) {
                bool vload = vec > 1 && c.strides[k][rank - 1] == 1;
                std::string e = vload ? "r" + std::to_string(k) + "[u][" + j + "]" : "r" + std::to_string(k) + "[u]";
                text += (k > n_out ? ", " : "") + from_storage(operands[k].dtype, e);
            }
            return text + ")";
        };
        if (vec > 1) {
            ss << "            V" << o << " out" << o << ";\n#pragma unroll\n            for (int j = 0; j < VEC; j++) {\n";
            ss << "                out" << o << "[j] = " << to_storage(operands[o].dtype, call("j")) << ";\n            }\n";
            int64_t os = c.strides[o][rank - 1];
            if (os == 1) ss << "            " << store_stmt("V" + os_name, "p" + os_name + " + off[u][" + os_name + "]", "out" + os_name, is_streaming(operands[o])) << "\n";
            else {
                // output is not contiguous along the vector axis (never picked by pick_vec, kept for completeness)
                ss << "#pragma unroll\n            for (int j = 0; j < VEC; j++) p" << o << "[off[u][" << o << "] + (idx_t) j * (idx_t) " << os << "] = out" << o << "[j];\n";
            }
        } else {
            ss << "            p" << o << "[off[u][" << o << "]] = " << to_storage(operands[o].dtype, call("0")) << ";\n";
        }
    }
    ss << "        }\n    }\n}\n";

    spec.source = ss.str();
    spec.grid = ceil_div_u32(total_vecs, 256 * unroll);
    std::ostringstream note;
    note << "rank=" << rank << " vec=" << vec << " unroll=" << unroll << " idx=" << (idx64 ? 64 : 32);
    if (n_out > 1) note << " outputs=" << n_out;
    spec.strategy = note.str();
    return spec;
}

// ------------------------------------------------------------------------------------------------ reduce kernel

// How many slices of the reduced index to fold side by side: none while there is a workgroup per compute unit or
// little to read per workgroup; else enough for about four workgroups per compute unit, each with 64 KB or more.
size_t reduce_parts(size_t blocks, size_t block_bytes, size_t most) {
    if (blocks >= 256 || block_bytes < ((size_t) 512 << 10)) return 1;
    const size_t wanted = (1024 + blocks - 1) / blocks, by_work = block_bytes / ((size_t) 64 << 10);
    return std::max<size_t>(1, std::min({wanted, by_work, most, (size_t) 1024}));
}

KernelSpec make_reduce_kernel(const KernelOperand &input, const KernelOperand &output, const std::vector<size_t> &axes,
                              ReduceOp rop, const ScalarExpr *pre, ReduceSplit *split, const ReduceStat *stat) {
    const auto &ishape = input.shape.shape();
    // the folded values have the type of the output; with a prologue the loaded operand may be of another type
    const DType dtype = output.dtype, in_dtype = input.dtype;
    if (stat) {
        // pairs of floats out of floats or halves (a prologue gives floats)
        KN_ASSERT(dtype == DType::F32 && (pre ? pre->nodes.back().dtype == DType::F32 : (in_dtype == DType::F32 || in_dtype == DType::F16)));
        rop = ReduceOp::Sum;
    } else {
        KN_ASSERT(pre ? pre->nodes.back().dtype == dtype : in_dtype == dtype);
    }

    // split axes into kept and reduced
    std::vector<size_t> kept_shape, red_shape;
    std::vector<int64_t> kept_in, kept_out, red_in;
    size_t out_axis = 0;
    for (size_t a = 0; a < ishape.size(); a++) {
        bool reduced = std::find(axes.begin(), axes.end(), a) != axes.end();
        if (reduced) {
            red_shape.push_back(ishape[a]);
            red_in.push_back(input.shape.strides()[a]);
        } else {
            KN_ASSERT(out_axis < output.shape.rank() && output.shape.shape()[out_axis] == ishape[a]);
            kept_shape.push_back(ishape[a]);
            kept_in.push_back(input.shape.strides()[a]);
            kept_out.push_back(output.shape.strides()[out_axis]);
            out_axis++;
        }
    }
    KN_ASSERT(out_axis == output.shape.rank());

    KernelSpec spec;
    spec.name = "kn_reduce";
    spec.n_ptrs = 2;
    size_t kept_size = concrete_size(kept_shape), red_size = concrete_size(red_shape);
    if (kept_size == 0) return spec;

    Collapsed kc = collapse_axes(kept_shape, {kept_out, kept_in}, true);
    // the reduction order is free: iterate with the smallest stride innermost
    Collapsed rc = collapse_axes(red_shape, {red_in}, true);

    int64_t min_kept = INT64_MAX, min_red = INT64_MAX;
    for (size_t a = 0; a < kc.rank(); a++) min_kept = std::min<int64_t>(min_kept, std::llabs(kc.strides[1][a]));
    for (size_t a = 0; a < rc.rank(); a++) min_red = std::min<int64_t>(min_red, std::llabs(rc.strides[0][a]));
    bool row = kc.rank() == 0 || rc.rank() == 0 || min_red <= min_kept;

    std::vector<KernelOperand> both{input, output};
    bool idx64 = !fits_i32(both, std::max(kept_size, red_size) + 4096);
    size_t es = dtype_bytes(in_dtype);

    const char *T = compute_type(dtype);
    DScalar identity = reduce_identity(rop, dtype);
    BinaryOp bop = rop == ReduceOp::Prod ? BinaryOp::Mul : rop == ReduceOp::Min ? BinaryOp::Min
                   : rop == ReduceOp::Max ? BinaryOp::Max : BinaryOp::Add;

    std::ostringstream ss;
    emit_header(ss, idx64, 2);
    ss << "typedef " << storage_type(dtype) << " S;\ntypedef " << storage_type(in_dtype) << " SI;\n";
    if (!stat) ss << "typedef " << T << " T;\ntypedef T X;\n";
    else ss << "typedef float X;\n#define KN_PLANE ((idx_t) " << stat->plane << ")\n";
    // the value that is folded: the loaded element, or an elementwise expression of it
    ss << "KN_DEV X kn_pre(" << compute_type(in_dtype) << " x1) {\n";
    if (pre) {
        std::string res = emit_expr(ss, *pre, "y", [&](size_t operand) {
            KN_ASSERT(operand == 1);
            return std::string("x1");
        });
        ss << "    return " << res << ";\n}\n";
    } else {
        ss << "    return x1;\n}\n";
    }
    if (!stat) {
        ss << "KN_DEV T kn_f(T a, T b) { return " << binary_expr(bop, dtype, "a", "b") << "; }\n";
        ss << "KN_DEV T kn_identity() { return " << identity.to_c_str() << "; }\n";
        ss << "KN_DEV void kn_acc(T &t, X x) { t = kn_f(t, x); }\n";
        ss << "KN_DEV T kn_post(T v) { return "
           << (rop == ReduceOp::Mean ? "v / (float) " + std::to_string(red_size) + ".0f" : std::string("v")) << "; }\n";
        ss << "KN_DEV void kn_store(S *at, T v) { *at = " << to_storage(dtype, "kn_post(v)") << "; }\n";
    } else if (stat->kind == ReduceStat::MaxSumExp) {
        // a: the maximum so far, b: sum of exp(x - a). An element of -inf adds nothing (a row of nothing else ends as
        // (-inf, 0) and its results as NaN, like exp(-inf - -inf)); +inf or NaN make the sum NaN, like exp(inf - inf).
        ss << R"KN(struct T { float a, b; };
KN_DEV T kn_identity() { return T{-KN_INF, 0.0f}; }
KN_DEV void kn_acc(T &t, float x) {
    const float e = __expf(-fabsf(x - t.a));  // (a term of a sum of many: the hardware's 2^x, a few 1e-7 off)
    const float b = x > t.a ? t.b * e + 1.0f : t.b + e;
    t.b = x == -KN_INF ? t.b : (x == KN_INF ? __builtin_nanf("") : b);
    t.a = fmaxf(t.a, x);
}
KN_DEV T kn_f(T p, T q) {
    const float m = fmaxf(p.a, q.a);
    const float sp = p.a == m ? p.b : p.b * expf(p.a - m), sq = q.a == m ? q.b : q.b * expf(q.a - m);
    return T{m, sp + sq};
}
KN_DEV void kn_store(S *at, T v) { at[0] = v.a; at[KN_PLANE] = 1.0f / v.b; }
)KN";
    } else {
        // (count, mean, M2): Welford per element, the reciprocal of the count from the hardware (the mean moves by
        // d / n, so an ulp of 1 / n is an ulp of a correction); Chan's combination between accumulators
        ss << R"KN(struct T { float n, mean, m2; };
KN_DEV T kn_identity() { return T{0.0f, 0.0f, 0.0f}; }
KN_DEV void kn_acc(T &t, float x) {
    t.n += 1.0f;
    const float d = x - t.mean;
    t.mean += d * __frcp_rn(t.n);
    t.m2 += d * (x - t.mean);
}
KN_DEV T kn_f(T p, T q) {
    const float n = p.n + q.n;
    if (n == 0.0f) return p;
    const float d = q.mean - p.mean, r = q.n / n;
    return T{n, p.mean + d * r, (p.m2 + q.m2) + d * d * (p.n * r)};
}
)KN";
        ss << "KN_DEV void kn_store(S *at, T v) { at[0] = v.mean; at[KN_PLANE] = 1.0f / sqrtf(v.m2 / v.n + " << DScalar::f32(stat->eps).to_c_str() << "); }\n";
    }

    const std::string preamble = ss.str();
    const bool may_split = split != nullptr && dtype != DType::Bool;
    size_t parts = 1;
    std::ostringstream note;
    if (row) {
        // ---- a group of G lanes folds one output element, lanes stride over the (contiguous) reduced index
        size_t vec = 1;
        if (rc.rank() > 0 && rc.strides[0].back() == 1) {
            for (vec = 16 / es; vec > 1; vec /= 2) {
                bool ok = rc.shape.back() % vec == 0 && input.offset_bytes % (int64_t) (vec * es) == 0;
                for (size_t a = 0; a + 1 < rc.rank(); a++) ok &= rc.strides[0][a] % (int64_t) vec == 0;
                for (size_t a = 0; a < kc.rank(); a++) ok &= kc.strides[1][a] % (int64_t) vec == 0;
                if (ok) break;
            }
        }
        // Many short rows whose length is no multiple of the vector (sums over 33 floats of [2097152, 33]): lanes that
        // walk a row each would fetch single elements, a line per few lanes. The rows of a dense input follow each other
        // in memory, so a workgroup takes 256 of them as ONE contiguous run with 128 bit loads into LDS and every
        // thread folds a row from there.
        const size_t row_bytes = red_size * es;
        if (!stat && vec == 1 && 16 / es > 1 && kc.rank() == 1 && rc.rank() == 1 && rc.strides[0][0] == 1 && kc.strides[0][0] == 1 &&
            kc.strides[1][0] == (int64_t) red_size && red_size >= 3 && row_bytes <= 240 && kept_size >= 16384 &&
            input.offset_bytes % 16 == 0 && kept_size * red_size < (1ull << 31)) {
            const size_t ve = 16 / es;
            ss << vec_type_decl("V", in_dtype, ve);
            ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_reduce(KnPtrs ptrs) {\n";
            ss << "    const SI *in = (const SI *) ptrs.p[0];\n    S *out = (S *) ptrs.p[1];\n";
            ss << "    __shared__ __attribute__((aligned(16))) SI tile[" << 256 * red_size << "];\n";
            ss << "    const idx_t row0 = (idx_t) blockIdx.x * (idx_t) 256;\n";
            ss << "    const idx_t rows = (idx_t) " << kept_size << " - row0 < (idx_t) 256 ? (idx_t) " << kept_size << " - row0 : (idx_t) 256;\n";
            ss << "    const SI *src = in + row0 * (idx_t) " << red_size << ";\n";
            ss << "    const idx_t elems = rows * (idx_t) " << red_size << ", vecs = elems / (idx_t) " << ve << ";\n";
            // (256 rows are a whole number of vectors: every run starts on a 16 byte boundary)
            ss << "#pragma unroll 4\n    for (idx_t v = (idx_t) threadIdx.x; v < vecs; v += (idx_t) 256) ((V *) tile)[v] = "
               << load_expr("V", "(const V *) src + v", is_streaming(input)) << ";\n";
            ss << "    for (idx_t e = vecs * (idx_t) " << ve << " + (idx_t) threadIdx.x; e < elems; e += (idx_t) 256) tile[e] = src[e];\n";
            ss << "    __syncthreads();\n";
            ss << "    if ((idx_t) threadIdx.x < rows) {\n        T acc = kn_identity();\n";
            ss << "        const SI *mine = tile + (idx_t) threadIdx.x * (idx_t) " << red_size << ";\n";
            ss << "#pragma unroll 11\n        for (int j = 0; j < " << red_size << "; j++) acc = kn_f(acc, kn_pre(" << from_storage(in_dtype, "mine[j]") << "));\n";
            ss << "        out[row0 + (idx_t) threadIdx.x] = " << to_storage(dtype, "kn_post(acc)") << ";\n    }\n}\n";
            spec.block = 256;
            spec.grid = ceil_div_u32(kept_size, 256);
            spec.source = ss.str();
            note << "short rows, 256 at a time through LDS";
            spec.strategy = note.str();
            if (split) split->parts = 1;
            return spec;
        }
        size_t red_vecs = red_size / vec;
        size_t G = red_vecs >= 2048 ? 256 : red_vecs >= 128 ? 64 : red_vecs >= 16 ? 16 : 1;
        size_t block = 256, rows_per_block = block / G;
        const size_t blocks = (kept_size + rows_per_block - 1) / rows_per_block;
        if (may_split) parts = reduce_parts(blocks, red_size * rows_per_block * es, red_vecs / (4 * G));
        // every slice is `chunk` vectors of the reduced index long (the last one may be shorter, none is empty)
        const size_t chunk = (red_vecs + parts - 1) / parts;
        parts = (red_vecs + chunk - 1) / chunk;
        size_t iters = (chunk + G - 1) / G;
        std::vector<size_t> rdims = rc.shape;
        std::vector<std::vector<int64_t>> rstrides = rc.strides;
        if (rc.rank() > 0) {
            rdims.back() /= vec;
            rstrides[0].back() *= (int64_t) vec;
        }
        if (vec > 1) ss << vec_type_decl("V", in_dtype, vec);
        ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_reduce(KnPtrs ptrs) {\n";
        ss << "    const SI *in = (const SI *) ptrs.p[0];\n    S *out = (S *) ptrs.p[1];\n";
        if (G == 256) ss << "    __shared__ T lds[4];\n";
        if (parts > 1) {
            ss << "    const idx_t part = (idx_t) blockIdx.x / (idx_t) " << blocks << ", blk = (idx_t) blockIdx.x % (idx_t) " << blocks << ";\n";
            ss << "    const idx_t r0 = part * (idx_t) " << chunk << ";\n";
            ss << "    const idx_t r1 = r0 + (idx_t) " << chunk << " < (idx_t) " << red_vecs << " ? r0 + (idx_t) " << chunk << " : (idx_t) " << red_vecs << ";\n";
        } else {
            ss << "    const idx_t blk = (idx_t) blockIdx.x, r0 = 0, r1 = (idx_t) " << red_vecs << ";\n";
        }
        ss << "    const idx_t row = blk * (idx_t) " << rows_per_block << " + (idx_t) (threadIdx.x / " << G << ");\n";
        ss << "    const idx_t lane = (idx_t) (threadIdx.x % " << G << ");\n";
        if (G != 256) ss << "    if (row >= (idx_t) " << kept_size << ") return;\n";
        ss << "    idx_t o_out = 0, o_in = 0;\n";
        emit_decompose(ss, "    ", "row", kc.shape, kc.strides, {"o_out", "o_in"});
        ss << "    T acc[4] = {kn_identity(), kn_identity(), kn_identity(), kn_identity()};\n";
        ss << (iters <= 32 ? "#pragma unroll\n" : "#pragma unroll 8\n");
        ss << "    for (idx_t i = 0; i < (idx_t) " << iters << "; i++) {\n";
        ss << "        const idx_t r = r0 + lane + i * (idx_t) " << G << ";\n";
        ss << "        if (r < r1) {\n            idx_t o = o_in;\n";
        emit_decompose(ss, "            ", "r", rdims, rstrides, {"o"});
        if (vec > 1) {
            ss << "            const V v = " << load_expr("V", "in + o", is_streaming(input)) << ";\n#pragma unroll\n";
            ss << "            for (int j = 0; j < " << vec << "; j++) kn_acc(acc[(i + j) & 3], " << "kn_pre(" + from_storage(in_dtype, "v[j]") + ")" << ");\n";
        } else {
            ss << "            kn_acc(acc[i & 3], " << "kn_pre(" + from_storage(in_dtype, "in[o]") + ")" << ");\n";
        }
        ss << "        }\n    }\n";
        ss << "    T total = kn_f(kn_f(acc[0], acc[1]), kn_f(acc[2], acc[3]));\n";
        if (G == 256) ss << "    total = kn_block_reduce<4>(total, kn_f, lds);\n";
        else if (G > 1) ss << "    total = kn_group_reduce<" << G << ">(total, kn_f);\n";
        if (parts > 1) ss << "    if (lane == 0) ((T *) ptrs.p[1])[part * (idx_t) " << kept_size << " + row] = total;\n}\n";
        else ss << "    if (lane == 0) kn_store(out + o_out, total);\n}\n";
        spec.block = (uint32_t) block;
        spec.grid = ceil_div_u32(blocks * parts, 1);
        note << "row G=" << G << " vec=" << vec << " iters=" << iters;
    } else {
        // ---- every thread owns VEC neighbouring kept elements and walks the reduced index; TY slices of the
        // reduction run side by side and are combined through LDS
        size_t vec = 1;
        if (kc.strides[1].back() == 1 && kc.strides[0].back() == 1) {
            for (vec = 16 / es; vec > 1; vec /= 2) {
                // (pairs are stored float by float: only the loads are vectors then)
                bool ok = kc.shape.back() % vec == 0 && input.offset_bytes % (int64_t) (vec * es) == 0 &&
                          (stat || output.offset_bytes % (int64_t) (vec * dtype_bytes(dtype)) == 0);
                for (size_t a = 0; a + 1 < kc.rank(); a++)
                    ok &= (stat || kc.strides[0][a] % (int64_t) vec == 0) && kc.strides[1][a] % (int64_t) vec == 0;
                for (size_t a = 0; a < rc.rank(); a++) ok &= rc.strides[0][a] % (int64_t) vec == 0;
                if (ok) break;
            }
        }
        size_t kept_vecs = kept_size / vec;
        size_t TX = 64;
        while (TX > 1 && TX / 2 >= kept_vecs) TX /= 2;
        size_t TY = 256 / TX;
        while (TY > 1 && TY > red_size) TY /= 2;
        // with plenty of independent outputs there is no need to split the reduction
        if (kept_vecs >= 256 * 1024) { TX = 256; TY = 1; }
        size_t block = TX * TY;
        const size_t blocks = (kept_vecs + TX - 1) / TX;
        if (may_split) parts = reduce_parts(blocks, red_size * TX * vec * es, red_size / (4 * TY));
        const size_t chunk = (red_size + parts - 1) / parts;
        parts = (red_size + chunk - 1) / chunk;
        std::vector<size_t> kdims = kc.shape;
        std::vector<std::vector<int64_t>> kstrides = kc.strides;
        kdims.back() /= vec;
        kstrides[0].back() *= (int64_t) vec;
        kstrides[1].back() *= (int64_t) vec;
        if (vec > 1) ss << vec_type_decl("V", in_dtype, vec) << (stat ? std::string() : vec_type_decl("VO", dtype, vec));
        ss << "extern \"C\" __global__ __launch_bounds__(" << block << ") void kn_reduce(KnPtrs ptrs) {\n";
        ss << "    const SI *in = (const SI *) ptrs.p[0];\n    S *out = (S *) ptrs.p[1];\n";
        if (TY > 1) ss << "    __shared__ T lds[" << TY << "][" << vec << "][" << TX << "];\n";
        ss << "    const idx_t tx = (idx_t) (threadIdx.x % " << TX << "), ty = (idx_t) (threadIdx.x / " << TX << ");\n";
        if (parts > 1) {
            ss << "    const idx_t part = (idx_t) blockIdx.x / (idx_t) " << blocks << ", blk = (idx_t) blockIdx.x % (idx_t) " << blocks << ";\n";
            ss << "    const idx_t r0 = part * (idx_t) " << chunk << ";\n";
            ss << "    const idx_t r1 = r0 + (idx_t) " << chunk << " < (idx_t) " << red_size << " ? r0 + (idx_t) " << chunk << " : (idx_t) " << red_size << ";\n";
        } else {
            ss << "    const idx_t blk = (idx_t) blockIdx.x, r0 = 0, r1 = (idx_t) " << red_size << ";\n";
        }
        ss << "    const idx_t kv = blk * (idx_t) " << TX << " + tx;\n";
        ss << "    const bool valid = kv < (idx_t) " << kept_vecs << ";\n";
        ss << "    idx_t o_out = 0, o_in = 0;\n";
        ss << "    T acc[" << vec << "];\n    for (int j = 0; j < " << vec << "; j++) acc[j] = kn_identity();\n";
        ss << "    if (valid) {\n";
        emit_decompose(ss, "        ", "kv", kdims, kstrides, {"o_out", "o_in"});
        ss << "#pragma unroll 4\n        for (idx_t r = r0 + ty; r < r1; r += (idx_t) " << TY << ") {\n            idx_t o = o_in;\n";
        emit_decompose(ss, "            ", "r", rc.shape, rc.strides, {"o"});
        if (vec > 1) {
            ss << "            const V v = " << load_expr("V", "in + o", is_streaming(input)) << ";\n#pragma unroll\n";
            ss << "            for (int j = 0; j < " << vec << "; j++) kn_acc(acc[j], " << "kn_pre(" + from_storage(in_dtype, "v[j]") + ")" << ");\n";
        } else {
            ss << "            kn_acc(acc[0], " << "kn_pre(" + from_storage(in_dtype, "in[o]") + ")" << ");\n";
        }
        ss << "        }\n    }\n";
        if (TY > 1) {
            ss << "    for (int j = 0; j < " << vec << "; j++) lds[ty][j][tx] = acc[j];\n    __syncthreads();\n";
            ss << "    if (ty == 0 && valid) {\n        for (int j = 0; j < " << vec << "; j++) {\n            T t = lds[0][j][tx];\n";
            ss << "            for (int s = 1; s < " << TY << "; s++) t = kn_f(t, lds[s][j][tx]);\n            acc[j] = t;\n        }\n";
        } else {
            ss << "    if (valid) {\n";
        }
        if (parts > 1) {
            ss << "        T *slot = (T *) ptrs.p[1] + (part * (idx_t) " << kept_vecs << " + kv) * (idx_t) " << vec << ";\n";
            ss << "        for (int j = 0; j < " << vec << "; j++) slot[j] = acc[j];\n";
        } else if (vec > 1 && !stat) {
            ss << "        VO o;\n        for (int j = 0; j < " << vec << "; j++) o[j] = " << to_storage(dtype, "kn_post(acc[j])") << ";\n";
            ss << "        *(VO *) (out + o_out) = o;\n";
        } else {
            ss << "        for (int j = 0; j < " << vec << "; j++) kn_store(out + o_out + j, acc[j]);\n";
        }
        ss << "    }\n}\n";
        spec.block = (uint32_t) block;
        spec.grid = ceil_div_u32(blocks * parts, 1);
        note << "col TX=" << TX << " TY=" << TY << " vec=" << vec;
    }
    if (parts > 1) {
        // the second kernel folds the slices of every result and applies the mean's division: one thread per result
        // (neighbouring threads read neighbouring partial results), or a wave per result when there are few results
        // and many slices, each lane folding every 64th slice before the lanes are combined
        note << " parts=" << parts;
        const size_t FG = kept_size <= 4096 && parts >= 16 ? 64 : 1;
        std::ostringstream fs;
        fs << preamble;
        fs << "extern \"C\" __global__ __launch_bounds__(256) void kn_reduce_final(KnPtrs ptrs) {\n";
        fs << "    const T *part = (const T *) ptrs.p[0];\n    S *out = (S *) ptrs.p[1];\n";
        fs << "    const idx_t i = ((idx_t) blockIdx.x * (idx_t) 256 + (idx_t) threadIdx.x) / (idx_t) " << FG << ";\n";
        fs << "    const idx_t lane = (idx_t) (threadIdx.x % " << FG << ");\n";
        fs << "    if (i >= (idx_t) " << kept_size << ") return;\n    idx_t o_out = 0;\n";
        emit_decompose(fs, "    ", "i", kc.shape, {kc.strides[0]}, {"o_out"});
        if (FG > parts) fs << "    T acc = lane < (idx_t) " << parts << " ? part[lane * (idx_t) " << kept_size << " + i] : kn_identity();\n#pragma unroll 8\n";
        else fs << "    T acc = part[lane * (idx_t) " << kept_size << " + i];\n#pragma unroll 8\n";
        fs << "    for (idx_t s = lane + (idx_t) " << FG << "; s < (idx_t) " << parts << "; s += (idx_t) " << FG << ") acc = kn_f(acc, part[s * (idx_t) " << kept_size << " + i]);\n";
        if (FG > 1) fs << "    acc = kn_group_reduce<" << FG << ">(acc, kn_f);\n";
        fs << "    if (lane == 0) kn_store(out + o_out, acc);\n}\n";
        split->parts = parts;
        split->kept_size = kept_size;
        split->partial_dtype = dtype == DType::F16 ? DType::F32 : dtype;
        split->partial_words = !stat ? 1 : (stat->kind == ReduceStat::MaxSumExp ? 2 : 3);
        split->final.name = "kn_reduce_final";
        split->final.n_ptrs = 2;
        split->final.block = 256;
        split->final.grid = ceil_div_u32(kept_size * FG, 256);
        split->final.source = fs.str();
        split->final.strategy = "fold of " + std::to_string(parts) + " partial results" + (FG > 1 ? ", a wave per result" : "");
    }
    spec.source = ss.str();
    spec.strategy = note.str();
    return spec;
}

// ------------------------------------------------------------------------------------------------ row kernels

// the row statistic of kind Reduce out of the folded value `m` (the mean divides, like the reduce kernel's last step)
std::string stat_expr_of(bool rowred, ReduceOp rop, size_t size) {
    return rowred && rop == ReduceOp::Mean ? "m / (float) " + std::to_string(size) + ".0f" : std::string("m");
}

KernelSpec make_row_kernel(const RowKernelDesc &desc) {
    const auto &ops = desc.operands;
    KN_ASSERT(ops.size() >= 2);
    const auto &shape = ops[0].shape.shape();
    size_t axis = desc.axis;
    KN_ASSERT(axis < shape.size());
    size_t size = shape[axis];

    std::vector<size_t> static_shape;
    std::vector<std::vector<int64_t>> static_strides(ops.size());
    std::vector<int64_t> axis_strides;
    for (size_t k = 0; k < ops.size(); k++) {
        KN_ASSERT(ops[k].shape.shape() == shape, "all operands of a row kernel must have the same shape");
        axis_strides.push_back(ops[k].shape.strides()[axis]);
    }
    for (size_t a = 0; a < shape.size(); a++) {
        if (a == axis) continue;
        static_shape.push_back(shape[a]);
        for (size_t k = 0; k < ops.size(); k++) static_strides[k].push_back(ops[k].shape.strides()[a]);
    }

    const bool softmax = desc.kind == RowKernelDesc::Softmax, rowred = desc.kind == RowKernelDesc::Reduce;
    const ReduceOp rop = desc.reduce_op;
    KN_ASSERT(!rowred || rop == ReduceOp::Sum || rop == ReduceOp::Mean || rop == ReduceOp::Max || rop == ReduceOp::Min);
    // identity and fold of the first reduction over the row
    const bool fold_max = softmax || (rowred && rop == ReduceOp::Max), fold_min = rowred && rop == ReduceOp::Min;
    const char *identity = fold_max ? "-KN_INF" : (fold_min ? "KN_INF" : "0.0f");
    const char *fold_fn = fold_max ? "kn_max" : (fold_min ? "kn_min" : "kn_add");
    KernelSpec spec;
    spec.name = softmax ? "kn_softmax" : (rowred ? "kn_rowreduce" : "kn_layernorm");
    spec.n_ptrs = ops.size();
    size_t static_size = concrete_size(static_shape);
    if (static_size == 0 || size == 0) return spec;
    // the normalised value is x * (1 / denom) instead of x / denom: one division per row, at most one ulp apart
    constexpr bool use_rcp = true;

    Collapsed sc = collapse_axes(static_shape, static_strides, true);

    // vector width along the normalised axis
    size_t max_bytes = 1;
    for (auto &op : ops) max_bytes = std::max(max_bytes, dtype_bytes(op.dtype));
    size_t vec = 16 / max_bytes;
    for (; vec > 1; vec /= 2) {
        bool ok = size % vec == 0;
        for (size_t k = 0; k < ops.size() && ok; k++) {
            int64_t as = axis_strides[k];
            if (as != 0 && as != 1) ok = false;
            if (k == 0 && as != 1) ok = false;
            if (as == 1) {
                size_t es = dtype_bytes(ops[k].dtype);
                ok &= ops[k].offset_bytes % (int64_t) (vec * es) == 0;
                for (size_t a = 0; a < sc.rank(); a++) ok &= sc.strides[k][a] % (int64_t) vec == 0;
            }
        }
        if (ok) break;
    }
    // Rows whose length is no multiple of the vector, or that start at any element (rows of 50257 floats follow each
    // other at every alignment): still whole vectors. Vectors may start at any element, and the last vector of a row
    // ends with the row, overlapping the one before it: the elements it repeats are left out of the sums and written
    // twice with the same value. Only for rows that are held in registers, from a few vectors per lane on.
    bool ragged = false;
    if (vec == 1 && 16 / max_bytes > 1 && size >= 4096 && size <= (size_t) 64 * 1024) {
        bool ok = true;
        for (size_t k = 0; k < ops.size() && ok; k++) ok = k == 0 ? axis_strides[k] == 1 : (axis_strides[k] == 0 || axis_strides[k] == 1);
        if (ok) {
            vec = 16 / max_bytes;
            ragged = true;
        }
    }
    const size_t rem = size % vec;  // elements of the last vector that are its own (0: all of them)
    size_t nv = (size + vec - 1) / vec;
    // G lanes share a row; the row stays in registers when every lane holds at most MAX_ITEMS vectors: 64 elements,
    // which the kernel keeps as floats. (With 16 vectors of 8 halves a lane of 1024 would hold 128 and spill: f16
    // [1046, 128256] 396 us held against 240 us read again per pass; single elements held up to 64 instead of 16: f32
    // rows of 50257 486 us read again per pass.)
    const size_t MAX_ITEMS = std::max<size_t>(1, 64 / vec);
    size_t G = 1024;
    for (size_t g : {1, 4, 16, 64, 256, 1024}) {
        size_t per_lane = (nv + g - 1) / g;
        constexpr size_t wave_items = 4;
        constexpr size_t block_items = 8;
        size_t limit = g == 1024 ? MAX_ITEMS : g == 256 ? block_items : g == 64 ? wave_items : g == 1 ? 2 : 4;
        if (per_lane <= limit) {
            G = g;
            break;
        }
    }
    size_t items = (nv + G - 1) / G;
    bool cached = items <= MAX_ITEMS;
    if (!cached) spec.row_access = KernelSpec::RowsStreamed;
    constexpr size_t min_block = 256;  // (rows that span several waves get a workgroup each: G is 256 or 1024 then)
    size_t block = std::max<size_t>(G, min_block);
    size_t rows_per_block = block / G;
    size_t nw = G / 64;  // waves per row when a row spans several waves
    bool idx64 = !fits_i32(ops, std::max(static_size, size) + 4096);

    std::ostringstream ss;
    emit_header(ss, idx64, ops.size());
    for (size_t k = 0; k < ops.size(); k++) {
        ss << "typedef " << storage_type(ops[k].dtype) << " S" << k << ";\n";
        if (vec > 1) ss << vec_type_decl("V" + std::to_string(k), ops[k].dtype, vec, ragged);
    }
    // which operands feed the prologue / epilogue
    std::vector<bool> in_pre(ops.size(), false), in_post(ops.size(), false);
    for (auto &n : desc.pre.nodes)
        if (n.kind == ScalarNode::Load) in_pre.at(n.operand) = true;
    for (auto &n : desc.post.nodes)
        if (n.kind == ScalarNode::Load && n.operand != SIZE_MAX) in_post.at(n.operand) = true;

    auto emit_fn = [&](const char *name, const ScalarExpr &expr, const std::vector<bool> &used, bool with_norm, DType result) {
        ss << "KN_DEV " << compute_type(result) << " " << name << "(";
        bool first = true;
        if (with_norm) {
            ss << "float xn";
            first = false;
        }
        for (size_t k = 1; k < ops.size(); k++) {
            if (!used[k]) continue;
            ss << (first ? "" : ", ") << compute_type(ops[k].dtype) << " x" << k;
            first = false;
        }
        ss << ") {\n";
        std::string res = emit_expr(ss, expr, "y", [&](size_t operand) {
            return operand == SIZE_MAX ? std::string("xn") : "x" + std::to_string(operand);
        });
        ss << "    return " << res << ";\n}\n";
    };
    // f16 rows are held, reduced and normalised in f32; the normalised value is rounded to f16 before the epilogue
    const DType row_dtype = desc.pre.nodes.back().dtype;
    KN_ASSERT(row_dtype == DType::F32 || row_dtype == DType::F16);
    KN_ASSERT(desc.post.nodes.back().dtype == ops[0].dtype);
    // The exponential of a softmax over halves: the hardware's 2^x on x * log2(e), a few 1e-6 off relative for the
    // arguments that do not vanish in f16, where a result is rounded to 11 bits anyway. The library's expf is about
    // twenty instructions per element, which is what rows of halves then wait for, not memory (f16 [13421, 10000]
    // 121.8 -> 87.3 us, rows of 128256 249 -> 139 us). f32 rows keep expf.
    ss << "#define kn_exp(x) " << (row_dtype == DType::F16 ? "__expf(x)" : "expf(x)") << "\n";
    emit_fn("kn_pre", desc.pre, in_pre, false, row_dtype);
    emit_fn("kn_post", desc.post, in_post, true, ops[0].dtype);

    // The normalised axis is not the contiguous one, a kept axis is (a softmax over the channels of [n, c, h, w]):
    // lanes that walk along the axis would each touch a line of their own. Here TX neighbouring lanes take TX
    // neighbouring columns instead, so that every load of a wave is a run of whole lines, TY threads share a column
    // (every TY-th position of the axis each, in registers when those are few, else read again per pass) and
    // combine their statistics through LDS.
    if (sc.rank() >= 1 && axis_strides[0] != 1 && sc.strides[0].back() == 1 && sc.shape.back() >= 16 && size > 1) {
        const size_t inner = sc.shape.back();
        size_t n_pre = 0;
        for (size_t k = 1; k < ops.size(); k++) n_pre += in_pre[k] ? 1 : 0;
        size_t TX = 64, TY = 4, items = (size + 3) / 4, threads = 256;
        bool held = false;
        for (size_t tx : {64, 32, 16}) {  // fewer columns per workgroup: more threads, so more registers, per column
            const size_t ty = 256 / tx, per_thread = (size + ty - 1) / ty;
            if (per_thread * std::max<size_t>(n_pre, 1) <= 32) {
                TX = tx, TY = ty, items = per_thread, held = true;
                break;
            }
        }
        // A run of less than a cache line per row of lanes (16 or 32 halves, 16 floats), or a column too long for 256
        // threads: a workgroup of 1024 threads holds four times as much, a whole line per row of lanes. (f16
        // [64, 512, 32, 32] along axis 1: 61.0 -> 27.1 us; f32 [8, 1000, 4096] along axis 1, read three times before:
        // 94.3 -> 60.7 us; runs of two lines per row of lanes on 1024 threads where 256 threads manage one: 113 -> 123 us.)
        const size_t elem_bytes = dtype_bytes(ops[1].dtype);
        if ((!held || TX * elem_bytes < 128) && sc.shape.back() >= 64) {
            for (size_t tx : {64, 32}) {
                const size_t ty = 1024 / tx, per_thread = (size + ty - 1) / ty;
                if (tx * elem_bytes >= 128 && per_thread * std::max<size_t>(n_pre, 1) <= 32) {
                    TX = tx, TY = ty, items = per_thread, held = true, threads = 1024;
                    break;
                }
            }
        }
        std::vector<size_t> outer_shape(sc.shape.begin(), sc.shape.end() - 1);
        if (!held) {
            // read again per pass: what counts is how many loads are in flight, so as many workgroups as the columns
            // give, up to four per compute unit, before whole lines per wave
            for (size_t tx : {64, 32, 16}) {
                TX = tx, TY = 256 / tx, items = (size + TY - 1) / TY;
                if (concrete_size(outer_shape) * ((inner + tx - 1) / tx) >= 1024) break;
            }
        }
        spec.row_access = held ? KernelSpec::RowsHeld : KernelSpec::ColumnsStreamed;
        const size_t column_blocks = (inner + TX - 1) / TX;
        std::vector<std::vector<int64_t>> outer_strides(ops.size());
        for (size_t k = 0; k < ops.size(); k++) outer_strides[k].assign(sc.strides[k].begin(), sc.strides[k].end() - 1);
        const size_t outer_size = concrete_size(outer_shape);
        const std::string L = "(idx_t) " + std::to_string(size);
        ss << "KN_DEV float kn_max(float a, float b) { return fmaxf(a, b); }\nKN_DEV float kn_add(float a, float b) { return a + b; }\n";
        ss << "KN_DEV float kn_min(float a, float b) { return fminf(a, b); }\n";
        ss << "#define TX " << TX << "\n#define TY " << TY << "\n#define ITEMS " << items << "\n";
        // every thread of a column ends up with the fold of the TY partial values, taken in the same order
        ss << "template<typename F> KN_DEV float kn_column_fold(float v, F f, float (*lds)[TX], int tx, int ty) {\n";
        ss << "    lds[ty][tx] = v;\n    __syncthreads();\n    v = lds[0][tx];\n";
        ss << "#pragma unroll\n    for (int s = 1; s < TY; s++) v = f(v, lds[s][tx]);\n    return v;\n}\n";
        ss << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void " << spec.name << "(KnPtrs ptrs) {\n";
        for (size_t k = 0; k < ops.size(); k++) ss << "    S" << k << " *p" << k << " = (S" << k << " *) ptrs.p[" << k << "];\n";
        ss << "    __shared__ float lds_m[TY][TX], lds_s[TY][TX];\n";
        ss << "    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;\n";
        ss << "    const idx_t col_raw = ((idx_t) blockIdx.x % (idx_t) " << column_blocks << ") * (idx_t) TX + (idx_t) tx;\n";
        ss << "    const bool col_ok = col_raw < (idx_t) " << inner << ";\n";
        ss << "    const idx_t col = col_ok ? col_raw : (idx_t) " << (inner - 1) << ";\n";
        ss << "    const idx_t outer = (idx_t) blockIdx.x / (idx_t) " << column_blocks << ";\n";
        ss << "    idx_t base[" << ops.size() << "];\n";
        for (size_t k = 0; k < ops.size(); k++) ss << "    base[" << k << "] = col * (idx_t) " << i64_str(sc.strides[k].back()) << ";\n";
        {
            std::vector<std::string> offs;
            for (size_t k = 0; k < ops.size(); k++) offs.push_back("base[" + std::to_string(k) + "]");
            emit_decompose(ss, "    ", "outer", outer_shape, outer_strides, offs);
        }
        auto at = [&](size_t k, const std::string &i) {
            return "p" + std::to_string(k) + "[base[" + std::to_string(k) + "] + " + i + " * (idx_t) " + i64_str(axis_strides[k]) + "]";
        };
        auto pre_of = [&](const std::function<std::string(size_t)> &operand) {
            std::string c = "kn_pre(";
            bool first = true;
            for (size_t k = 1; k < ops.size(); k++) {
                if (!in_pre[k]) continue;
                c += (first ? "" : ", ") + from_storage(ops[k].dtype, operand(k));
                first = false;
            }
            return c + ")";
        };
        auto store = [&](const std::string &indent, const std::string &i, const std::string &value) {
            std::string c = row_dtype == DType::F16 ? "kn_post(kn_r16(" + value + ")" : "kn_post(" + value;
            for (size_t k = 1; k < ops.size(); k++)
                if (in_post[k]) c += ", " + from_storage(ops[k].dtype, at(k, i));
            ss << indent << at(0, i) << " = " << to_storage(ops[0].dtype, c + ")") << ";\n";
        };
        const std::string fold_stmt = fold_max ? "m = fmaxf(m, v);" : fold_min ? "m = fminf(m, v);" : "m += v;";
        const std::string eps = DScalar::f32(desc.eps).to_c_str();
        ss << "    float m = " << identity << ", s = 0.0f;\n";
        if (held) {
            for (size_t k = 1; k < ops.size(); k++)
                if (in_pre[k]) ss << "    S" << k << " a" << k << "[ITEMS];\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n";
            ss << "        const idx_t i = (idx_t) ty + (idx_t) it * (idx_t) TY, ic = i < " << L << " ? i : " << L << " - 1;\n";
            for (size_t k = 1; k < ops.size(); k++)
                if (in_pre[k]) ss << "        a" << k << "[it] = " << at(k, "ic") << ";\n";
            ss << "    }\n    float x[ITEMS];\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = (idx_t) ty + (idx_t) it * (idx_t) TY;\n";
            ss << "        const float v = i < " << L << " ? " << pre_of([&](size_t k) { return "a" + std::to_string(k) + "[it]"; }) << " : " << identity << ";\n";
            ss << "        x[it] = v;\n        " << fold_stmt << "\n    }\n";
            ss << "    m = kn_column_fold(m, " << fold_fn << ", lds_m, tx, ty);\n";
            if (rowred) {
                ss << "    const float stat = " << stat_expr_of(rowred, rop, size) << ";\n";
                ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) x[it] = stat;\n";
            } else if (softmax) {
                ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = (idx_t) ty + (idx_t) it * (idx_t) TY;\n";
                ss << "        const float e = i < " << L << " ? kn_exp(x[it] - m) : 0.0f;\n        x[it] = e;\n        s += e;\n    }\n";
                ss << "    s = kn_column_fold(s, kn_add, lds_s, tx, ty);\n";
                ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) x[it] = x[it] / s;\n";
            } else {
                ss << "    const float mean = m / (float) " << size << ".0f;\n";
                ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = (idx_t) ty + (idx_t) it * (idx_t) TY;\n";
                ss << "        const float d = i < " << L << " ? x[it] - mean : 0.0f;\n        x[it] = d;\n        s += d * d;\n    }\n";
                ss << "    s = kn_column_fold(s, kn_add, lds_s, tx, ty);\n";
                ss << "    const float rdenom = 1.0f / sqrtf(s / (float) " << size << ".0f + " << eps << ");\n";
                ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) x[it] = x[it] * rdenom;\n";
            }
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = (idx_t) ty + (idx_t) it * (idx_t) TY;\n";
            ss << "        if (col_ok && i < " << L << ") {\n";
            store("            ", "i", "x[it]");
            ss << "        }\n    }\n}\n";
        } else {
            ss << "    const idx_t len = col_ok ? " << L << " : (idx_t) 0;\n";
            const std::string loop = "    for (idx_t i = (idx_t) ty; i < len; i += (idx_t) TY) {\n";
            const std::string loaded = pre_of([&](size_t k) { return at(k, "i"); });
            if (softmax) {
                // two passes, as for rows too long for registers: the sum of exponentials is kept relative to the
                // running maximum, and the threads of a column scale theirs to the column's maximum before adding
                ss << "#pragma unroll 8\n" << loop << "        const float v = " << loaded << ";\n";
                ss << "        if (v > m) { s *= kn_exp(m - v); m = v; }\n";
                ss << "        s += v == -KN_INF ? 0.0f : kn_exp(v - m);\n    }\n";
                ss << "    const float m_mine = m;\n";
                ss << "    m = kn_column_fold(m, " << fold_fn << ", lds_m, tx, ty);\n";
                ss << "    s = m_mine == -KN_INF ? s : s * kn_exp(m_mine - m);\n";
                ss << "    s = kn_column_fold(s, kn_add, lds_s, tx, ty);\n";
                ss << "#pragma unroll 8\n" << loop << "        const float v = " << loaded << ";\n";
                ss << "        const float r = kn_exp(v - m) / s;\n";
                store("        ", "i", "r");
                ss << "    }\n}\n";
            } else {
            ss << "#pragma unroll 8\n" << loop << "        const float v = " << loaded << ";\n        " << fold_stmt << "\n    }\n";
            ss << "    m = kn_column_fold(m, " << fold_fn << ", lds_m, tx, ty);\n";
            if (rowred) {
                ss << "    const float stat = " << stat_expr_of(rowred, rop, size) << ";\n";
                ss << "#pragma unroll 8\n" << loop;
                store("        ", "i", "stat");
                ss << "    }\n}\n";
            } else {
                if (!softmax) ss << "    const float mean = m / (float) " << size << ".0f;\n";
                ss << "#pragma unroll 8\n" << loop << "        const float v = " << loaded << ";\n";
                if (softmax) ss << "        s += kn_exp(v - m);\n    }\n";
                else ss << "        const float d = v - mean;\n        s += d * d;\n    }\n";
                ss << "    s = kn_column_fold(s, kn_add, lds_s, tx, ty);\n";
                if (!softmax) ss << "    const float denom = sqrtf(s / (float) " << size << ".0f + " << eps << ");\n";
                ss << "#pragma unroll 8\n" << loop << "        const float v = " << loaded << ";\n";
                ss << "        const float r = " << (softmax ? "kn_exp(v - m) / s" : "(v - mean) / denom") << ";\n";
                store("        ", "i", "r");
                ss << "    }\n}\n";
            }
            }
        }
        spec.source = ss.str();
        spec.block = (uint32_t) threads;
        spec.grid = ceil_div_u32(outer_size * column_blocks, 1);
        std::ostringstream note;
        note << (softmax ? "softmax" : (rowred ? "row statistic + elementwise" : "layernorm")) << " columns TX=" << TX << " TY=" << TY
             << " items=" << items << (held ? " cached" : (softmax ? " streamed twice" : " streamed"));
        if (threads != 256) note << " threads=" << threads;
        spec.strategy = note.str();
        return spec;
    }

    // Epilogue operands (gamma, beta, ...) are requested together with the row itself when they fit in registers,
    // so that their latency overlaps with the reductions instead of following them.
    size_t n_post = 0;
    for (size_t k = 1; k < ops.size(); k++) {
        if (!in_post[k]) continue;
        n_post++;
    }
    bool prefetch_post = cached && n_post > 0 && n_post * items * vec <= 64;
    // Which of them: the row and the operands requested with it should stay within 32 values per lane, or the
    // kernel needs more than the 64 registers that full occupancy allows ([8192, 4096] with gamma and beta: 47.1 us
    // with both held from the start, one wave per SIMD less; 43.2 us with gamma alone, 42.6 us without either).
    // The others are loaded where the epilogue uses them, after the statistics, into registers that are free by then.
    std::vector<bool> early(ops.size(), false);
    if (prefetch_post) {
        size_t held = items * vec;
        for (size_t k = 1; k < ops.size(); k++) {
            if (!in_post[k]) continue;
            const size_t need = axis_strides[k] == 1 ? items * vec * std::max<size_t>(dtype_bytes(ops[k].dtype), 4) / 4 : items;
            if (held + need <= 32) {
                early[k] = true;
                held += need;
            }
        }
    }
    // Epilogue operands that are the same for every row (gamma, beta) and together as large as the L1 cache: every
    // row would fetch them from L2 again, and those fetches queue up with the row itself ([8192, 4096]: 42.6 us without
    // them, 43.0 us with gamma, 47.3 us with gamma and beta). A workgroup then stages them in LDS once and walks over
    // `seq` rows, as long as enough workgroups remain to fill the chip.
    std::vector<bool> staged(ops.size(), false);
    size_t seq = 1, staged_bytes = 0;
    if (cached && vec > 1 && !ragged) {
        for (size_t k = 1; k < ops.size(); k++) {
            if (!in_post[k] || in_pre[k] || axis_strides[k] != 1) continue;
            bool invariant = true;
            for (size_t a = 0; a < sc.rank(); a++) invariant &= sc.strides[k][a] == 0;
            if (invariant) {
                staged[k] = true;
                staged_bytes += size * dtype_bytes(ops[k].dtype);
            }
        }
        // (measured with gamma and beta, the loads of the next row requested ahead: 43.4 us with 2 rows per workgroup,
        // 45.8 us with 4, 49.0 us with 8; 47.3 us with one row and the operands from L2)
        if (staged_bytes >= 24 * 1024 && staged_bytes <= 40 * 1024 && static_size % (rows_per_block * 2) == 0 &&
            static_size / (rows_per_block * 2) >= 1024)
            seq = 2;
        if (seq == 1) staged.assign(ops.size(), false);
        else prefetch_post = false;  // (registers that hold operands of the epilogue would be refilled for the next row too early)
    }
    // Rows and vector positions past the end are clamped for addressing and masked afterwards, so that the loads of
    // a row are straight-line code that the compiler can issue back to back (a branch per load would make every
    // load wait for the one before it).
    const bool check_row = static_size % (rows_per_block * seq) != 0;
    const bool check_i = cached && items * G != nv;

    ss << "#define VEC " << vec << "\n#define ITEMS " << items << "\n#define G " << G << "\n";
    // whether element j of vector position i is that vector's own (not a repeat of the vector before the row's last)
    if (ragged && rem != 0) ss << "#define KN_OWN(i, j) ((i) != (idx_t) " << (nv - 1) << " || (j) >= " << (vec - rem) << ")\n";
    ss << "KN_DEV float kn_max(float a, float b) { return fmaxf(a, b); }\nKN_DEV float kn_add(float a, float b) { return a + b; }\n";
    ss << "KN_DEV float kn_min(float a, float b) { return fminf(a, b); }\n";
    auto emit_fold = [&](const std::string &indent, const std::string &src) {
        if (fold_max) ss << indent << "for (int j = 0; j < VEC; j++) m = fmaxf(m, " << src << "[j]);\n";
        else if (fold_min) ss << indent << "for (int j = 0; j < VEC; j++) m = fminf(m, " << src << "[j]);\n";
        else ss << indent << "for (int j = 0; j < VEC; j++) m += " << src << "[j];\n";
    };
    // the row statistic of kind Reduce from the folded value `m` (like the post step of the reduce kernel)
    const std::string stat_expr = stat_expr_of(rowred, rop, size);
    ss << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << spec.name << "(KnPtrs ptrs) {\n";
    for (size_t k = 0; k < ops.size(); k++) ss << "    S" << k << " *p" << k << " = (S" << k << " *) ptrs.p[" << k << "];\n";
    // (statistics of consecutive rows of a workgroup alternate between two sets of slots: one barrier per exchange)
    if (nw > 1) ss << "    __shared__ float lds_m[" << nw << "], lds_s[" << nw << "], lds_st[" << 2 * nw * (seq > 1 ? 2 : 1) << "];\n";
    for (size_t k = 1; k < ops.size(); k++)
        if (staged[k]) ss << "    __shared__ V" << k << " lds_b" << k << "[" << nv << "];\n";
    ss << "    const idx_t lane = (idx_t) (threadIdx.x % G);\n";
    ss << "    idx_t base[" << ops.size() << "];\n    for (int k = 0; k < " << ops.size() << "; k++) base[k] = 0;\n";
    const std::string row0 = "((idx_t) blockIdx.x * (idx_t) " + std::to_string(rows_per_block) + " + (idx_t) (threadIdx.x / G))";
    auto emit_row_setup = [&](const std::string &into = "base") {
        std::vector<std::string> offs;
        for (size_t k = 0; k < ops.size(); k++) offs.push_back(into + "[" + std::to_string(k) + "]");
        if (check_row) ss << "    const idx_t rowc = row < (idx_t) " << static_size << " ? row : (idx_t) " << (static_size - 1) << ";\n";
        emit_decompose(ss, "    ", check_row ? "rowc" : "row", sc.shape, sc.strides, offs);
    };
    if (seq == 1) {
        ss << "    const idx_t row = " << row0 << ";\n";
        emit_row_setup();
    }
    // the reduction helper: over G lanes of a wave, or over the waves of the workgroup
    auto reduce = [&](const std::string &var, const char *f) {
        if (G == 1) return;
        if (nw > 1) ss << "    " << var << " = kn_block_reduce<" << nw << ">(" << var << ", " << f << ", lds_" << var << ");\n";
        else ss << "    " << var << " = kn_group_reduce<G>(" << var << ", " << f << ");\n";
    };
    // element offset along the axis of vector position `i` of operand k: the last vector of a ragged row ends with the row
    const bool overlap = ragged && rem != 0;
    auto axis_offset = [&](size_t k, const std::string &i) {
        if (axis_strides[k] == 0) return std::string("(idx_t) 0");
        if (!overlap) return i + " * (idx_t) " + i64_str(axis_strides[k] * (int64_t) vec);
        KN_ASSERT(axis_strides[k] == 1);
        return "(" + i + " == (idx_t) " + std::to_string(nv - 1) + " ? (idx_t) " + std::to_string(size - vec) + " : " + i + " * (idx_t) " + std::to_string(vec) + ")";
    };
    // the prologue operands of vector position `i` (in vector units along the axis): loaded into `a<k>`, either
    // declared on the spot or assigned to an element of a register array that was declared earlier (`slot`)
    std::string pre_base = "base";  // the row offsets that the prologue loads start from
    auto emit_pre_loads = [&](const std::string &indent, const std::string &i, const std::string &slot) {
        for (size_t k = 1; k < ops.size(); k++) {
            if (!in_pre[k]) continue;
            std::string o = "(" + pre_base + "[" + std::to_string(k) + "] + " + axis_offset(k, i) + ")";
            bool v = vec > 1 && axis_strides[k] == 1;
            std::string lhs = slot.empty() ? std::string("const ") + (v ? "V" : "S") + std::to_string(k) + " a" + std::to_string(k)
                                           : "a" + std::to_string(k) + "[" + slot + "]";
            if (v) ss << indent << lhs << " = "
                      << load_expr("V" + std::to_string(k), "p" + std::to_string(k) + " + " + o, cached && is_streaming(ops[k])) << ";\n";
            else ss << indent << lhs << " = p" << k << "[" << o << "];\n";
        }
    };
    // run the prologue on the loaded operands
    auto emit_pre_apply = [&](const std::string &indent, const std::string &dst, const std::string &slot) {
        const std::string pick = slot.empty() ? std::string() : "[" + slot + "]";
        ss << indent << "for (int j = 0; j < VEC; j++) " << dst << "[j] = kn_pre(";
        bool first = true;
        for (size_t k = 1; k < ops.size(); k++) {
            if (!in_pre[k]) continue;
            std::string e = "a" + std::to_string(k) + pick + ((vec > 1 && axis_strides[k] == 1) ? "[j]" : "");
            ss << (first ? "" : ", ") << from_storage(ops[k].dtype, e);
            first = false;
        }
        ss << ");\n";
    };
    auto emit_load_pre = [&](const std::string &indent, const std::string &i, const std::string &dst) {
        emit_pre_loads(indent, i, "");
        emit_pre_apply(indent, dst, "");
    };
    // run the epilogue on normalised values `src[j]` of vector position `i` and store
    // the epilogue operands of vector position `i`: loaded into `prefix<k>`, either declared on the spot or
    // assigned to an element of a register array that was declared earlier (`slot`)
    auto emit_post_loads = [&](const std::string &indent, const std::string &i, const std::string &slot) {
        for (size_t k = 1; k < ops.size(); k++) {
            if (!in_post[k] || (prefetch_post && early[k] == slot.empty())) continue;
            if (staged[k]) {
                ss << indent << "const V" << k << " b" << k << " = lds_b" << k << "[" << i << "];\n";
                continue;
            }
            std::string o = "(base[" + std::to_string(k) + "] + " + axis_offset(k, i) + ")";
            bool v = vec > 1 && axis_strides[k] == 1;
            std::string lhs = slot.empty() ? std::string("const ") + (v ? "V" : "S") + std::to_string(k) + " b" + std::to_string(k)
                                           : "b" + std::to_string(k) + "[" + slot + "]";
            if (v) ss << indent << lhs << " = " << load_expr("V" + std::to_string(k), "p" + std::to_string(k) + " + " + o, is_streaming(ops[k])) << ";\n";
            else ss << indent << lhs << " = p" << k << "[" << o << "];\n";
        }
    };
    auto emit_post_store = [&](const std::string &indent, const std::string &i, const std::string &src, const std::string &slot) {
        emit_post_loads(indent, i, "");  // (those not requested ahead)
        const std::string pick = slot.empty() ? std::string() : "[" + slot + "]";
        std::string o0 = "(base[0] + " + axis_offset(0, i) + ")";
        auto call = [&](const std::string &j) {
            std::string c = row_dtype == DType::F16 ? "kn_post(kn_r16(" + src + "[" + j + "])" : "kn_post(" + src + "[" + j + "]";
            for (size_t k = 1; k < ops.size(); k++) {
                if (!in_post[k]) continue;
                std::string e = "b" + std::to_string(k) + (early[k] ? pick : std::string()) + ((vec > 1 && axis_strides[k] == 1) ? "[" + j + "]" : "");
                c += ", " + from_storage(ops[k].dtype, e);
            }
            return to_storage(ops[0].dtype, c + ")");
        };
        if (vec > 1) {
            ss << indent << "V0 o;\n" << indent << "for (int j = 0; j < VEC; j++) o[j] = " << call("j") << ";\n";
            ss << indent << store_stmt("V0", "p0 + " + o0, "o", is_streaming(ops[0])) << "\n";
        } else {
            ss << indent << "p0[" << o0 << "] = " << call("0") << ";\n";
        }
    };

    const std::string valid = check_row ? std::string("(row < (idx_t) ") + std::to_string(static_size) + ")" : std::string("true");
    if (cached) {
        const std::string item_index = std::string("        const idx_t i = lane + (idx_t) it * (idx_t) G;\n") +
            (check_i ? "        const idx_t ic = i < (idx_t) " + std::to_string(nv) + " ? i : (idx_t) " + std::to_string(nv - 1) + ";\n"
                     : std::string("        const idx_t ic = i;\n"));
        for (size_t k = 1; k < ops.size(); k++) {
            const char *t = (vec > 1 && axis_strides[k] == 1) ? "V" : "S";
            if (in_pre[k]) ss << "    " << t << k << " a" << k << "[ITEMS];\n";
            if (in_post[k] && prefetch_post && early[k]) ss << "    " << t << k << " b" << k << "[ITEMS];\n";
        }
        auto emit_row_loads = [&]() {
            // every load of the row first, then the arithmetic
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n" << item_index;
            emit_pre_loads("        ", "ic", "it");
            if (prefetch_post) emit_post_loads("        ", "ic", "it");
            ss << "    }\n";
        };
        const std::string seq_row = "(" + row0 + " / (idx_t) " + std::to_string(rows_per_block) + ") * (idx_t) " +
                                    std::to_string(rows_per_block * seq) + " + (idx_t) (threadIdx.x / G)";
        if (seq > 1) {
            // the rows of this group one after another; the loads of row r + 1 are requested as soon as row r has
            // left the registers they arrive in, i.e. before its statistics
            for (size_t k = 1; k < ops.size(); k++)
                if (staged[k])
                    ss << "    for (idx_t i = (idx_t) threadIdx.x; i < (idx_t) " << nv << "; i += (idx_t) " << block << ") lds_b" << k
                       << "[i] = *(const V" << k << " *) (p" << k << " + i * (idx_t) " << vec << ");\n";
            ss << "    idx_t nbase[" << ops.size() << "];\n    for (int k = 0; k < " << ops.size() << "; k++) nbase[k] = 0;\n";
            ss << "    {\n    const idx_t row = " << seq_row << ";\n";
            emit_row_setup("nbase");
            ss << "    }\n";
            pre_base = "nbase";
            emit_row_loads();
            ss << "    __syncthreads();\n";
            ss << "    for (int rs = 0; rs < " << seq << "; rs++) {\n";
            ss << "    const idx_t row = " << seq_row << " + (idx_t) rs * (idx_t) " << rows_per_block << ";\n";
            ss << "    for (int k = 0; k < " << ops.size() << "; k++) base[k] = nbase[k];\n";
        } else {
            emit_row_loads();
        }
        ss << "    float x[ITEMS][VEC];\n";
        ss << "    float m = " << identity << ";\n";
        ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = lane + (idx_t) it * (idx_t) G;\n";
        emit_pre_apply("        ", "x[it]", "it");
        if (check_i)
            ss << "        if (!(i < (idx_t) " << nv << ")) for (int j = 0; j < VEC; j++) x[it][j] = " << identity << ";\n";
        if (overlap) {
            // the last vector repeats VEC - rem elements of the one before it: those stay out of the fold
            ss << "        {\n            float own[VEC];\n            for (int j = 0; j < VEC; j++) own[j] = KN_OWN(i, j) ? x[it][j] : " << identity << ";\n";
            emit_fold("            ", "own");
            ss << "        }\n";
        } else {
            emit_fold("        ", "x[it]");
        }
        ss << "    }\n";
        if (seq > 1) {
            ss << "    if (rs + 1 < " << seq << ") {\n    const idx_t row = " << seq_row << " + (idx_t) (rs + 1) * (idx_t) " << rows_per_block << ";\n";
            ss << "    for (int k = 0; k < " << ops.size() << "; k++) nbase[k] = 0;\n";
            emit_row_setup("nbase");
            emit_row_loads();
            ss << "    }\n";
            pre_base = "base";
        }
        // layernorm with the same number of elements in every lane: per-lane mean and centred sum of squares,
        // combined pairwise in a single pass over the lanes instead of one pass for the mean and one for the
        // variance (one barrier instead of two when a row spans several waves)
        const bool one_pass = !softmax && !rowred && !check_i && !overlap && G > 1;
        if (!one_pass) reduce("m", fold_fn);
        if (!rowred) ss << "    float s = 0.0f;\n";
        if (rowred) {
            ss << "    const float stat = " << stat_expr << ";\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        for (int j = 0; j < VEC; j++) x[it][j] = stat;\n    }\n";
        } else if (softmax) {
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = lane + (idx_t) it * (idx_t) G;\n";
            ss << "        for (int j = 0; j < VEC; j++) {\n            const float e = (i < (idx_t) " << nv << ") ? kn_exp(x[it][j] - m) : 0.0f;\n";
            ss << "            x[it][j] = e;\n            s += " << (overlap ? "KN_OWN(i, j) ? e : 0.0f" : "e") << ";\n        }\n    }\n";
            reduce("s", "kn_add");
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        for (int j = 0; j < VEC; j++) x[it][j] = x[it][j] / s;\n    }\n";
        } else if (one_pass) {
            const size_t cnt = items * vec;
            ss << "    float mean = m / (float) " << cnt << ".0f;\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n";
            ss << "        for (int j = 0; j < VEC; j++) {\n            const float d = x[it][j] - mean;\n            s += d * d;\n        }\n    }\n";
            if (nw > 1) ss << "    kn_block_stats<" << nw << ">(mean, s, (float) " << cnt << ".0f, lds_st" << (seq > 1 ? " + (rs & 1) * " + std::to_string(2 * nw) : std::string()) << ");\n";
            else ss << "    kn_group_stats<G>(mean, s, (float) " << cnt << ".0f);\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        for (int j = 0; j < VEC; j++) x[it][j] = x[it][j] - mean;\n    }\n";
        } else {
            ss << "    const float mean = m / (float) " << size << ".0f;\n";
            ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = lane + (idx_t) it * (idx_t) G;\n";
            ss << "        for (int j = 0; j < VEC; j++) {\n            const float d = (i < (idx_t) " << nv << ") ? (x[it][j] - mean) : 0.0f;\n";
            ss << "            x[it][j] = d;\n            s += " << (overlap ? "KN_OWN(i, j) ? d * d : 0.0f" : "d * d") << ";\n        }\n    }\n";
            reduce("s", "kn_add");
        }
        if (!softmax && !rowred) {
            ss << "    const float denom = sqrtf(s / (float) " << size << ".0f + " << DScalar::f32(desc.eps).to_c_str() << ");\n";
            if (use_rcp) ss << "    const float rdenom = 1.0f / denom;\n#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        for (int j = 0; j < VEC; j++) x[it][j] = x[it][j] * rdenom;\n    }\n";
            else ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        for (int j = 0; j < VEC; j++) x[it][j] = x[it][j] / denom;\n    }\n";
        }
        ss << "#pragma unroll\n    for (int it = 0; it < ITEMS; it++) {\n        const idx_t i = lane + (idx_t) it * (idx_t) G;\n";
        std::string guard;
        if (check_i) guard = "i < (idx_t) " + std::to_string(nv);
        if (check_row) guard += (guard.empty() ? "" : " && ") + valid;
        ss << "        " << (guard.empty() ? std::string() : "if (" + guard + ") ") << "{\n";
        emit_post_store("            ", "i", "x[it]", prefetch_post ? "it" : "");
        ss << "        }\n    }\n";
        // (the slots of the other reductions are reused by the next row: everybody has to be done reading them)
        if (seq > 1) ss << (nw > 1 && !one_pass ? "    __syncthreads();\n" : "") << "    }\n";
        ss << "}\n";
    } else {
        // rows too long for registers: stream the row three times (the re-reads come from cache), a softmax twice
        ss << "    float t[VEC];\n";
        ss << "    float m = " << identity << ";\n";
        const std::string walk = "    if (" + valid + ")\n#pragma unroll 4\n    for (idx_t i = lane; i < (idx_t) " + std::to_string(nv) + "; i += (idx_t) G) {\n";
        if (softmax) {
            // Maximum and sum of exponentials in one pass: a lane's sum is kept relative to the largest value it has
            // seen and scaled down when a larger one comes; the lanes' sums are scaled to the row's maximum before
            // they are added. (A -inf adds nothing also while the maximum itself is still -inf, where the difference
            // would be a NaN; a NaN poisons the sum either way, as it does in three passes.)
            ss << "    float s = 0.0f;\n" << walk;
            emit_load_pre("        ", "i", "t");
            ss << "        float vm = t[0];\n        for (int j = 1; j < VEC; j++) vm = fmaxf(vm, t[j]);\n";
            ss << "        if (vm > m) { s *= kn_exp(m - vm); m = vm; }\n";
            ss << "        for (int j = 0; j < VEC; j++) s += t[j] == -KN_INF ? 0.0f : kn_exp(t[j] - m);\n    }\n";
            ss << "    const float m_lane = m;\n";
            reduce("m", fold_fn);
            ss << "    s = m_lane == -KN_INF ? s : s * kn_exp(m_lane - m);\n";
            reduce("s", "kn_add");
            ss << walk;
            emit_load_pre("        ", "i", "t");
            ss << "        for (int j = 0; j < VEC; j++) t[j] = kn_exp(t[j] - m) / s;\n";
            emit_post_store("        ", "i", "t", "");
            ss << "    }\n}\n";
            spec.source = ss.str();
            spec.block = (uint32_t) block;
            spec.grid = ceil_div_u32(static_size, rows_per_block * seq);
            std::ostringstream note;
            note << "softmax G=" << G << " vec=" << vec << " items=" << items << " streamed twice";
            spec.strategy = note.str();
            return spec;
        }
        ss << "    if (" << valid << ") for (idx_t i = lane; i < (idx_t) " << nv << "; i += (idx_t) G) {\n";
        emit_load_pre("        ", "i", "t");
        emit_fold("        ", "t");
        ss << "    }\n";
        reduce("m", fold_fn);
        if (rowred) {
            ss << "    const float stat = " << stat_expr << ";\n";
            ss << "    if (" << valid << ") for (idx_t i = lane; i < (idx_t) " << nv << "; i += (idx_t) G) {\n";
            ss << "        for (int j = 0; j < VEC; j++) t[j] = stat;\n";
            emit_post_store("        ", "i", "t", "");
            ss << "    }\n}\n";
        } else {
            if (!softmax) ss << "    const float mean = m / (float) " << size << ".0f;\n";
            ss << "    float s = 0.0f;\n";
            ss << "    if (" << valid << ") for (idx_t i = lane; i < (idx_t) " << nv << "; i += (idx_t) G) {\n";
            emit_load_pre("        ", "i", "t");
            if (softmax) ss << "        for (int j = 0; j < VEC; j++) s += kn_exp(t[j] - m);\n";
            else ss << "        for (int j = 0; j < VEC; j++) { const float d = t[j] - mean; s += d * d; }\n";
            ss << "    }\n";
            reduce("s", "kn_add");
            if (!softmax) ss << "    const float denom = sqrtf(s / (float) " << size << ".0f + " << DScalar::f32(desc.eps).to_c_str() << ");\n";
            ss << "    if (" << valid << ") for (idx_t i = lane; i < (idx_t) " << nv << "; i += (idx_t) G) {\n";
            emit_load_pre("        ", "i", "t");
            if (softmax) ss << "        for (int j = 0; j < VEC; j++) t[j] = kn_exp(t[j] - m) / s;\n";
            else ss << "        for (int j = 0; j < VEC; j++) t[j] = (t[j] - mean) / denom;\n";
            emit_post_store("        ", "i", "t", "");
            ss << "    }\n}\n";
        }
    }

    spec.source = ss.str();
    spec.block = (uint32_t) block;
    spec.grid = ceil_div_u32(static_size, rows_per_block * seq);
    std::ostringstream note;
    note << (softmax ? "softmax" : (rowred ? "row statistic + elementwise" : "layernorm")) << " G=" << G << " vec=" << vec << " items=" << items << (cached ? " cached" : " streamed");
    if (ragged) note << " vectors at any element" << (rem != 0 ? ", last one overlapping" : "");
    if (seq > 1) note << " rows=" << seq;
    spec.strategy = note.str();
    return spec;
}

// ------------------------------------------------------------------------------------------------ gather kernel

KernelSpec make_gather_kernel(const KernelOperand &input, const KernelOperand &indices, const KernelOperand &output,
                              size_t axis) {
    KN_ASSERT(indices.shape.rank() == 1);
    KN_ASSERT(input.dtype == output.dtype);
    const auto &ishape = input.shape.shape();
    const auto &oshape = output.shape.shape();
    KN_ASSERT(ishape.size() == oshape.size() && axis < ishape.size());
    size_t n_idx = indices.shape.shape()[0];
    KN_ASSERT(oshape[axis] == n_idx);

    KernelSpec spec;
    spec.name = "kn_gather";
    spec.n_ptrs = 3;
    spec.block = 256;
    size_t total = concrete_size(oshape);
    if (total == 0) return spec;

    // iterate in output order: all output axes, the gathered one included
    std::vector<std::vector<int64_t>> strides(3);
    for (size_t a = 0; a < oshape.size(); a++) {
        strides[0].push_back(output.shape.strides()[a]);
        strides[1].push_back(a == axis ? 0 : input.shape.strides()[a]);
        strides[2].push_back(a == axis ? indices.shape.strides()[0] : 0);
    }
    Collapsed c = collapse_axes(oshape, strides, true);
    if (c.rank() == 0) {
        c.shape = {1};
        for (auto &s : c.strides) s = {0};
    }
    std::vector<KernelOperand> all{input, indices, output};
    bool idx64 = !fits_i32(all, total + 4096);

    // Rows that are gathered whole (an embedding lookup, a selection of channels): when the fastest axis of the
    // result is not the gathered one and contiguous on both sides, a thread moves 16 bytes of it at a time.
    const size_t last = c.rank() - 1, es = dtype_bytes(input.dtype);
    const int64_t gathered_stride = input.shape.strides()[axis];
    size_t vec = 1;
    if (c.strides[0][last] == 1 && c.strides[1][last] == 1 && c.strides[2][last] == 0) {
        for (vec = 16 / es; vec > 1; vec /= 2) {
            bool ok = c.shape[last] % vec == 0 && gathered_stride % (int64_t) vec == 0;
            ok &= input.offset_bytes % (int64_t) (vec * es) == 0 && output.offset_bytes % (int64_t) (vec * es) == 0;
            for (size_t a = 0; a < last; a++) ok &= c.strides[0][a] % (int64_t) vec == 0 && c.strides[1][a] % (int64_t) vec == 0;
            if (ok) break;
        }
    }
    if (vec > 1) {
        c.shape[last] /= vec;
        c.strides[0][last] = c.strides[1][last] = (int64_t) vec;
    }
    // A gather along the contiguous axis of the input (the moves of a policy picked out of its planes): lanes that
    // read `in[row, index[j]]` touch a cache line each. With enough rows, and at least a quarter of a row wanted,
    // a workgroup stages the row in LDS with whole vectors and gathers from there.
    const size_t row_len = ishape[axis], rows = total / n_idx;
    if (c.strides[2][last] != 0 && c.shape[last] == n_idx && gathered_stride == 1 && row_len * es <= 65536 && rows >= 128 &&
        n_idx * 4 >= row_len && n_idx >= 64 && n_idx < ((size_t) 1 << 30)) {
        size_t rvec = 16 / es;
        for (; rvec > 1; rvec /= 2) {
            bool ok = row_len % rvec == 0 && input.offset_bytes % (int64_t) (rvec * es) == 0;
            for (size_t a = 0; a < last; a++) ok &= c.strides[1][a] % (int64_t) rvec == 0;
            if (ok) break;
        }
        std::vector<size_t> outer(c.shape.begin(), c.shape.begin() + (ptrdiff_t) last);
        std::vector<std::vector<int64_t>> outer_strides{
            std::vector<int64_t>(c.strides[0].begin(), c.strides[0].begin() + (ptrdiff_t) last),
            std::vector<int64_t>(c.strides[1].begin(), c.strides[1].begin() + (ptrdiff_t) last)};
        std::ostringstream ss;
        emit_header(ss, idx64, 3);
        ss << "typedef " << storage_type(input.dtype) << " S;\ntypedef " << dtype_c_name(indices.dtype) << " I;\n";
        if (rvec > 1) ss << vec_type_decl("V", input.dtype, rvec);
        else ss << "typedef S V;\n";
        ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_gather(KnPtrs ptrs) {\n";
        ss << "    const S *in = (const S *) ptrs.p[0];\n    const I *indices = (const I *) ptrs.p[1];\n    S *out = (S *) ptrs.p[2];\n";
        ss << "    __shared__ __attribute__((aligned(16))) S row[" << row_len << "];\n";
        ss << "    const idx_t r = (idx_t) blockIdx.x;\n    idx_t o_out = 0, o_in = 0;\n";
        emit_decompose(ss, "    ", "r", outer, outer_strides, {"o_out", "o_in"});
        ss << "    for (int i = threadIdx.x * " << rvec << "; i < " << row_len << "; i += " << 256 * rvec << ")\n";
        ss << "        *(V *) (row + i) = *(const V *) (in + o_in + i);\n";
        ss << "    __syncthreads();\n";
        ss << "    for (int j = threadIdx.x; j < " << n_idx << "; j += 256) {\n";
        ss << "        const I index = indices[(idx_t) j * (idx_t) " << c.strides[2][last] << "];\n";
        ss << "        S value = 0;\n";
        if (dtype_is_signed(indices.dtype))
            ss << "        if (index >= 0 && (unsigned long long) index < " << row_len << "ull)";
        else
            ss << "        if ((unsigned long long) index < " << row_len << "ull)";
        ss << " value = row[index];\n";
        ss << "        out[o_out + (idx_t) j * (idx_t) " << c.strides[0][last] << "] = value;\n    }\n}\n";
        spec.source = ss.str();
        spec.grid = ceil_div_u32(rows, 1);
        spec.strategy = "rank=" + std::to_string(c.rank()) + " rows staged in LDS vec=" + std::to_string(rvec);
        return spec;
    }
    const size_t items = total / vec;
    // four independent loads per thread once there are workgroups to spare
    const size_t unroll = items >= ((size_t) 1 << 20) ? 4 : 1;
    const bool nt = is_streaming(output);

    std::ostringstream ss;
    emit_header(ss, idx64, 3);
    ss << "typedef " << storage_type(input.dtype) << " S;\ntypedef " << dtype_c_name(indices.dtype) << " I;\n";
    if (vec > 1) ss << vec_type_decl("V", input.dtype, vec);
    else ss << "typedef S V;\n";
    ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_gather(KnPtrs ptrs) {\n";
    ss << "    const S *in = (const S *) ptrs.p[0];\n    const I *indices = (const I *) ptrs.p[1];\n    S *out = (S *) ptrs.p[2];\n";
    ss << "    const idx_t first = (idx_t) blockIdx.x * " << 256 * unroll << " + (idx_t) threadIdx.x;\n";
    ss << "    V value[" << unroll << "];\n    idx_t where[" << unroll << "];\n";
    ss << "#pragma unroll\n    for (int u = 0; u < " << unroll << "; u++) {\n";
    ss << "        const idx_t flat = first + u * 256;\n";
    ss << "        __builtin_memset(&value[u], 0, sizeof(V));\n        where[u] = -1;\n";
    ss << "        if (flat < (idx_t) " << items << ") {\n";
    ss << "            idx_t o_out = 0, o_in = 0, o_idx = 0;\n";
    emit_decompose(ss, "            ", "flat", c.shape, c.strides, {"o_out", "o_in", "o_idx"});
    ss << "            const I index = indices[o_idx];\n            where[u] = o_out;\n";
    if (dtype_is_signed(indices.dtype))
        ss << "            if (index >= 0 && (unsigned long long) index < " << ishape[axis] << "ull)";
    else
        ss << "            if ((unsigned long long) index < " << ishape[axis] << "ull)";
    ss << " value[u] = *(const V *) (in + o_in + (idx_t) index * (idx_t) " << gathered_stride << ");\n";
    ss << "        }\n    }\n";
    ss << "#pragma unroll\n    for (int u = 0; u < " << unroll << "; u++)\n";
    ss << "        if (first + u * 256 < (idx_t) " << items << ") " << store_stmt("V", "out + where[u]", "value[u]", nt) << "\n}\n";

    spec.source = ss.str();
    spec.grid = ceil_div_u32(items, 256 * unroll);
    spec.strategy = "rank=" + std::to_string(c.rank()) + " vec=" + std::to_string(vec) + " unroll=" + std::to_string(unroll);
    return spec;
}

}  // namespace kn
