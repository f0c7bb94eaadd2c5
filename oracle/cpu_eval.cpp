// ORACLE - TEST INFRASTRUCTURE ONLY. Nothing in the shipped library or package may call into this file.
//
// A CPU restatement of the reference's graph evaluator `cpu_eval_graph` (kn-graph/src/cpu.rs:20-88) and of the
// scalar semantics it relies on (kn-graph/src/graph.rs:1597-1815, kn-graph/src/dtype.rs:323-391). It takes a
// serialised graph (the flat format of kyanite_amd/csrc/serialize.cpp, parsed here independently), a batch size
// and dense row-major inputs, walks the values in topological order and materialises every value densely.
//
// Only `tests/`, the smoke check and the `cpu_baseline` leg of the benchmark use it, as the checker and as a
// timed baseline. It is single threaded, like the reference (ndarray without a BLAS backend).
//
// What pins it (see tests/test_oracle_*.py): the expected vectors the reference's own tests hold (elementwise
// sweep values, softplus, casts, flip, repeat, gather, linear, affine / batch-norm folding, clamp, broadcast add,
// chained scalar ops, complex multiply), the four ONNX + check-data fixtures of the reference's tests
// (kn-cuda-eval/tests/data, whole-graph outputs reproduced to 2e-7 ... 2e-6 relative) and closed forms / numpy
// brute force for what those leave open.
// Parity unpinned at the bit level: the accumulation order inside ndarray's `sum_axis` / `mean_axis` / `dot`
// (third party, not in the reference tree) - softmax, layernorm, conv and matmul here accumulate each output
// element sequentially in f32, which is tolerance-equal, not bit-equal, to the reference's CPU path.
//
// Deviation: binary operations, matmul and conv on f64 operands are evaluated (the reference panics for f64
// pairs, dtype.rs:460-483); F16 (absent from the reference) loads f16, computes and accumulates in f32 and rounds the
// result of every operation of the graph to f16 once (reduce, mean, softmax, layernorm and matmul included).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace {

enum DT : uint8_t { F32 = 0, F64, I8, I16, I32, I64, U8, U16, U32, U64, BOOL, F16 };
enum OP : uint8_t { Input = 0, Constant, View, Broadcast, Permute, Slice, Flip, Gather, Concat, Conv, MatMul, Unary, Binary, Softmax, Layernorm, Reduce };
enum UN : uint8_t { Abs = 0, Neg, Sin, Cos, Exp, Log, Sqrt, Sigmoid, Tanh, Erf, Mish, Softplus, ValueCast, BitCast };
enum BI : uint8_t { Add = 0, Sub, Mul, Div, Min, Max, Pow };
enum RE : uint8_t { Sum = 0, Mean, Prod, RMax, RMin };

[[noreturn]] void die(const std::string &msg) { throw std::runtime_error(msg); }

size_t dt_bytes(uint8_t t) {
    switch (t) {
        case F32: case I32: case U32: return 4;
        case F64: case I64: case U64: return 8;
        case I16: case U16: case F16: return 2;
        default: return 1;
    }
}

// ---- half precision, round to nearest even
uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mant = x & 0x7fffffu;
    int exp = (int) ((x >> 23) & 0xff);
    if (exp == 0xff) return (uint16_t) (sign | 0x7c00u | (mant ? 0x200u | (mant >> 13) : 0));
    exp = exp - 127 + 15;
    if (exp >= 31) return (uint16_t) (sign | 0x7c00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t) sign;
        mant |= 0x800000u;
        uint32_t shift = (uint32_t) (14 - exp), half = mant >> shift, rem = mant & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t) (sign | half);
    }
    uint32_t half = ((uint32_t) exp << 10) | (mant >> 13), rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t) (sign | half);
}
float h2f(uint16_t h) {
    uint32_t sign = ((uint32_t) h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, x;
    if (exp == 0) {
        if (!mant) x = sign;
        else {
            int e = -1;
            do { e++; mant <<= 1; } while (!(mant & 0x400u));
            x = sign | ((uint32_t) (127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7f800000u | (mant << 13);
    else x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}
struct half_t {
    uint16_t bits;
};

struct Tensor {
    uint8_t dtype = F32;
    std::vector<size_t> shape;
    std::shared_ptr<std::vector<uint8_t>> data;
    size_t len() const {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        return n;
    }
    template <typename T> T *ptr() { return (T *) data->data(); }
    template <typename T> const T *ptr() const { return (const T *) data->data(); }
    static Tensor make(uint8_t dtype, std::vector<size_t> shape) {
        Tensor t;
        t.dtype = dtype;
        t.shape = std::move(shape);
        t.data = std::make_shared<std::vector<uint8_t>>(t.len() * dt_bytes(dtype), 0);
        return t;
    }
};

struct SizeV {
    uint64_t factor;
    uint32_t exp;
    size_t eval(uint64_t batch) const {
        size_t r = factor;
        for (uint32_t k = 0; k < exp; k++) r *= batch;
        return r;
    }
};

struct Node {
    uint8_t dtype, op;
    std::vector<SizeV> shape;
    std::vector<uint32_t> inputs;
    std::vector<size_t> axes;
    size_t index = 0, start = 0, end = 0, step = 1;
    Tensor constant;
    size_t conv[8] = {0};  // stride_y, stride_x, padding_y, padding_x, kernel_h, kernel_w, output_h, output_w
    uint8_t sub = 0, cast_to = 0;
    float eps = 0;
};

struct Reader {
    const uint8_t *p;
    size_t len, pos = 0;
    void raw(void *d, size_t n) {
        if (pos + n > len) die("oracle: truncated graph blob");
        memcpy(d, p + pos, n);
        pos += n;
    }
    uint8_t u8() { uint8_t v; raw(&v, 1); return v; }
    uint32_t u32() { uint32_t v; raw(&v, 4); return v; }
    uint64_t u64() { uint64_t v; raw(&v, 8); return v; }
    float f32() { float v; raw(&v, 4); return v; }
};

struct ParsedGraph {
    std::vector<Node> nodes;
    std::vector<uint32_t> inputs, outputs;
};

ParsedGraph parse(const uint8_t *blob, size_t len) {
    Reader r{blob, len};
    if (r.u32() != 0x47484e4bu) die("oracle: bad magic");
    if (r.u32() != 1) die("oracle: bad version");
    ParsedGraph g;
    uint32_t n = r.u32();
    for (uint32_t i = 0; i < n; i++) {
        Node nd;
        nd.dtype = r.u8();
        uint32_t rank = r.u32();
        for (uint32_t k = 0; k < rank; k++) {
            SizeV s;
            s.factor = r.u64();
            s.exp = r.u32();
            nd.shape.push_back(s);
        }
        nd.op = r.u8();
        switch (nd.op) {
            case Input: nd.index = r.u32(); break;
            case Constant: {
                uint64_t bytes = r.u64();
                std::vector<size_t> dims;
                for (auto &s : nd.shape) dims.push_back(s.factor);
                nd.constant = Tensor::make(nd.dtype, dims);
                if (bytes != nd.constant.data->size()) die("oracle: constant size mismatch");
                r.raw(nd.constant.data->data(), bytes);
                break;
            }
            case View: case Broadcast: nd.inputs = {r.u32()}; break;
            case Permute: {
                nd.inputs = {r.u32()};
                uint32_t k = r.u32();
                for (uint32_t j = 0; j < k; j++) nd.axes.push_back(r.u32());
                break;
            }
            case Slice:
                nd.inputs = {r.u32()};
                nd.axes = {r.u32()};
                nd.start = r.u64(); nd.end = r.u64(); nd.step = r.u64();
                break;
            case Flip: case Softmax:
                nd.inputs = {r.u32()};
                nd.axes = {r.u32()};
                break;
            case Gather: {
                uint32_t in = r.u32();
                nd.axes = {r.u32()};
                uint32_t idx = r.u32();
                nd.inputs = {in, idx};
                break;
            }
            case Concat: {
                uint32_t k = r.u32();
                for (uint32_t j = 0; j < k; j++) nd.inputs.push_back(r.u32());
                nd.axes = {r.u32()};
                break;
            }
            case Conv: {
                uint32_t a = r.u32(), b = r.u32();
                nd.inputs = {a, b};
                for (int k = 0; k < 8; k++) nd.conv[k] = r.u64();
                break;
            }
            case MatMul: {
                uint32_t a = r.u32(), b = r.u32();
                nd.inputs = {a, b};
                break;
            }
            case Unary:
                nd.inputs = {r.u32()};
                nd.sub = r.u8();
                nd.cast_to = r.u8();
                break;
            case Binary: {
                uint32_t a = r.u32(), b = r.u32();
                nd.inputs = {a, b};
                nd.sub = r.u8();
                break;
            }
            case Layernorm:
                nd.inputs = {r.u32()};
                nd.axes = {r.u32()};
                nd.eps = r.f32();
                break;
            case Reduce: {
                nd.inputs = {r.u32()};
                uint32_t k = r.u32();
                for (uint32_t j = 0; j < k; j++) nd.axes.push_back(r.u32());
                nd.sub = r.u8();
                break;
            }
            default: die("oracle: unknown operation");
        }
        uint32_t id_len = r.u32();
        r.pos += id_len;
        g.nodes.push_back(std::move(nd));
    }
    uint32_t ni = r.u32();
    for (uint32_t k = 0; k < ni; k++) g.inputs.push_back(r.u32());
    uint32_t no = r.u32();
    for (uint32_t k = 0; k < no; k++) g.outputs.push_back(r.u32());
    return g;
}

// ---- typed dispatch
template <typename F>
auto dispatch(uint8_t dtype, F f) {
    switch (dtype) {
        case F32: return f((float *) nullptr);
        case F64: return f((double *) nullptr);
        case I8: return f((int8_t *) nullptr);
        case I16: return f((int16_t *) nullptr);
        case I32: return f((int32_t *) nullptr);
        case I64: return f((int64_t *) nullptr);
        case U8: return f((uint8_t *) nullptr);
        case U16: return f((uint16_t *) nullptr);
        case U32: return f((uint32_t *) nullptr);
        case U64: return f((uint64_t *) nullptr);
        case BOOL: return f((bool *) nullptr);
        case F16: return f((half_t *) nullptr);
    }
    die("oracle: bad dtype");
}

std::vector<int64_t> dense_strides(const std::vector<size_t> &shape) {
    std::vector<int64_t> s(shape.size());
    int64_t next = 1;
    for (size_t a = shape.size(); a-- > 0;) {
        s[a] = next;
        next *= (int64_t) shape[a];
    }
    return s;
}

// materialise a strided view densely; only the element size matters
Tensor gather_strided(const Tensor &src, const std::vector<size_t> &shape, const std::vector<int64_t> &strides, int64_t offset) {
    Tensor out = Tensor::make(src.dtype, shape);
    size_t es = dt_bytes(src.dtype), n = out.len(), rank = shape.size();
    if (n == 0) return out;
    std::vector<size_t> idx(rank, 0);
    const uint8_t *sp = src.data->data();
    uint8_t *dp = out.data->data();
    int64_t cur = offset;
    // fast path: innermost axis contiguous
    size_t inner = rank ? shape[rank - 1] : 1;
    bool inner_dense = rank == 0 || strides[rank - 1] == 1;
    for (size_t flat = 0; flat < n;) {
        if (inner_dense) {
            memcpy(dp + flat * es, sp + cur * (int64_t) es, inner * es);
            flat += inner;
            if (rank <= 1) break;
            for (size_t a = rank - 1; a-- > 0;) {
                idx[a]++;
                cur += strides[a];
                if (idx[a] < shape[a]) break;
                cur -= strides[a] * (int64_t) shape[a];
                idx[a] = 0;
            }
        } else {
            memcpy(dp + flat * es, sp + cur * (int64_t) es, es);
            flat++;
            for (size_t a = rank; a-- > 0;) {
                idx[a]++;
                cur += strides[a];
                if (idx[a] < shape[a]) break;
                cur -= strides[a] * (int64_t) shape[a];
                idx[a] = 0;
            }
        }
    }
    return out;
}

// ---- scalar semantics (graph.rs:1649-1735, :1791-1815)

double erf_as(double x) {
    // Abramowitz and Stegun; `signum` of a NaN is NaN, of +-0 is +-1
    static const double A[] = {1.0, 0.0705230784, 0.0422820123, 0.0092705272, 0.0001520143, 0.0002765672, 0.0000430638};
    double sign = std::isnan(x) ? x : (std::signbit(x) ? -1.0 : 1.0);
    double xa = std::fabs(x), d = 0;
    for (int i = 0; i < 7; i++) d += A[i] * std::pow(xa, i);  // powi
    return sign * (1.0 - 1.0 / std::pow(d, 16));
}

template <typename F>
F float_unary(uint8_t op, F x) {
    switch (op) {
        case Abs: return std::fabs(x);
        case Neg: return -x;
        case Sin: return std::sin(x);
        case Cos: return std::cos(x);
        case Exp: return std::exp(x);
        case Log: return std::log(x);
        case Sqrt: return std::sqrt(x);
        case Sigmoid: return (F) 1.0 / ((F) 1.0 + std::exp(-x));
        case Tanh: return std::tanh(x);
        case Erf: return (F) erf_as((double) x);
        case Mish: return x * std::tanh(std::log1p(std::exp(x)));
        case Softplus: {
            // Rust's f32::max ignores a NaN operand
            F relu = std::isnan(x) ? (F) 0 : (x > 0 ? x : (F) 0);
            return std::log1p(std::exp(-std::fabs(x))) + relu;
        }
    }
    die("oracle: not a float unary op");
}

// `x as i128` then truncation: saturating, NaN -> 0 (dtype.rs:326-337)
__int128 to_i128(double x) {
    if (std::isnan(x)) return 0;
    const double lim = 170141183460469231731687303715884105728.0;  // 2^127
    __int128 mx = (__int128) ((~(unsigned __int128) 0) >> 1);
    if (x >= lim) return mx;
    if (x < -lim) return -mx - 1;
    return (__int128) x;
}

template <typename T> struct Wide { };

template <typename T>
void load_wide(const T &v, double *yf, __int128 *yi) {
    if constexpr (std::is_same<T, half_t>::value) {
        float f = h2f(v.bits);
        *yf = f;
        *yi = to_i128(f);
    } else if constexpr (std::is_floating_point<T>::value) {
        *yf = (double) v;
        *yi = to_i128((double) v);
    } else if constexpr (std::is_same<T, bool>::value) {
        *yf = v ? 1.0 : 0.0;
        *yi = v ? 1 : 0;
    } else {
        *yf = (double) v;
        *yi = (__int128) v;
    }
}

template <typename T>
T store_wide(double yf, __int128 yi) {
    if constexpr (std::is_same<T, half_t>::value) return half_t{f2h((float) yf)};
    else if constexpr (std::is_same<T, float>::value) return (float) yf;
    else if constexpr (std::is_same<T, double>::value) return yf;
    else if constexpr (std::is_same<T, bool>::value) return yf != 0.0 || yi != 0;
    else return (T) (unsigned __int128) yi;  // wrapping truncation
}

Tensor eval_unary(const Node &nd, const Tensor &x, const std::vector<size_t> &out_shape) {
    Tensor out = Tensor::make(nd.dtype, out_shape);
    size_t n = out.len();
    if (nd.sub == ValueCast) {
        dispatch(x.dtype, [&](auto *sp) {
            using S = std::remove_pointer_t<decltype(sp)>;
            dispatch(nd.dtype, [&](auto *dp) {
                using D = std::remove_pointer_t<decltype(dp)>;
                const S *src = x.ptr<S>();
                D *dst = out.ptr<D>();
                for (size_t i = 0; i < n; i++) {
                    double yf;
                    __int128 yi;
                    load_wide<S>(src[i], &yf, &yi);
                    dst[i] = store_wide<D>(yf, yi);
                }
                return 0;
            });
            return 0;
        });
        return out;
    }
    if (nd.sub == BitCast) {
        if (dt_bytes(x.dtype) != dt_bytes(nd.dtype) || x.dtype == BOOL || nd.dtype == BOOL) die("oracle: invalid bitcast");
        memcpy(out.data->data(), x.data->data(), out.data->size());
        return out;
    }
    if (x.dtype == F32) {
        const float *s = x.ptr<float>();
        float *d = out.ptr<float>();
        for (size_t i = 0; i < n; i++) d[i] = float_unary<float>(nd.sub, s[i]);
    } else if (x.dtype == F64) {
        const double *s = x.ptr<double>();
        double *d = out.ptr<double>();
        for (size_t i = 0; i < n; i++) d[i] = float_unary<double>(nd.sub, s[i]);
    } else if (x.dtype == F16) {
        const uint16_t *s = x.ptr<uint16_t>();
        uint16_t *d = out.ptr<uint16_t>();
        for (size_t i = 0; i < n; i++) d[i] = f2h(float_unary<float>(nd.sub, h2f(s[i])));
    } else if ((nd.sub == Abs || nd.sub == Neg) && (x.dtype == I8 || x.dtype == I16 || x.dtype == I32 || x.dtype == I64)) {
        dispatch(x.dtype, [&](auto *tp) {
            using T = std::remove_pointer_t<decltype(tp)>;
            if constexpr (std::is_integral<T>::value && std::is_signed<T>::value) {
                using U = std::make_unsigned_t<T>;
                const T *s = x.ptr<T>();
                T *d = out.ptr<T>();
                for (size_t i = 0; i < n; i++) {
                    bool negate = nd.sub == Neg || s[i] < 0;
                    d[i] = negate ? (T) (U) ((U) 0 - (U) s[i]) : s[i];  // wrapping, as a release build does
                }
            }
            return 0;
        });
    } else {
        die("oracle: unary operation not supported on this dtype");
    }
    return out;
}

template <typename T>
T binary_scalar(uint8_t op, T l, T r) {
    if constexpr (std::is_same<T, bool>::value) {
        switch (op) {  // dtype.rs:726-757, Ord for min/max
            case Add: case Max: return l || r;
            case Mul: case Min: return l && r;
            case Sub: case Div: return l && !r;
        }
        die("oracle: unsupported bool op");
    } else if constexpr (std::is_floating_point<T>::value) {
        switch (op) {
            case Add: return l + r;
            case Sub: return l - r;
            case Mul: return l * r;
            case Div: return l / r;
            case Min: return std::isnan(l) ? r : (std::isnan(r) ? l : (l < r ? l : r));
            case Max: return std::isnan(l) ? r : (std::isnan(r) ? l : (l > r ? l : r));
            case Pow: return std::pow(l, r);
        }
        die("oracle: bad binary op");
    } else {
        using U = std::make_unsigned_t<T>;
        switch (op) {
            case Add: return (T) (U) ((U) l + (U) r);
            case Sub: return (T) (U) ((U) l - (U) r);
            case Mul: return (T) (U) ((uint64_t) (U) l * (uint64_t) (U) r);
            case Div:
                if (r == 0) die("oracle: attempt to divide by zero");
                if constexpr (std::is_signed<T>::value) {
                    if (r == (T) -1) return (T) (U) ((U) 0 - (U) l);
                }
                return (T) (l / r);
            case Min: return l < r ? l : r;
            case Max: return l > r ? l : r;
        }
        die("oracle: Pow is only supported for f32");
    }
}

Tensor eval_binary(const Node &nd, const Tensor &l, const Tensor &r) {
    if (l.dtype != r.dtype || l.shape != r.shape) die("oracle: binary operand mismatch");
    Tensor out = Tensor::make(nd.dtype, l.shape);
    size_t n = out.len();
    if (l.dtype == F16) {
        const uint16_t *a = l.ptr<uint16_t>(), *b = r.ptr<uint16_t>();
        uint16_t *d = out.ptr<uint16_t>();
        for (size_t i = 0; i < n; i++) d[i] = f2h(binary_scalar<float>(nd.sub, h2f(a[i]), h2f(b[i])));
        return out;
    }
    dispatch(l.dtype, [&](auto *tp) {
        using T = std::remove_pointer_t<decltype(tp)>;
        if constexpr (!std::is_same<T, half_t>::value) {
            const T *a = l.ptr<T>(), *b = r.ptr<T>();
            T *d = out.ptr<T>();
            for (size_t i = 0; i < n; i++) d[i] = binary_scalar<T>(nd.sub, a[i], b[i]);
        }
        return 0;
    });
    return out;
}

// C[i, j] += sum_k A[i, k] * B[k, j], every C element accumulated sequentially over k in the element type
template <typename T>
void gemm_acc(const T *a, const T *b, T *c, size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m; i++) {
        T *ci = c + i * n;
        for (size_t kk = 0; kk < k; kk++) {
            T av = a[i * k + kk];
            const T *bk = b + kk * n;
            for (size_t j = 0; j < n; j++) ci[j] += av * bk[j];
        }
    }
}

Tensor eval_matmul(const Tensor &l, const Tensor &r) {
    // cpu.rs:421-439
    if (l.shape.size() != 3 || r.shape.size() != 3 || l.shape[0] != r.shape[0] || l.shape[2] != r.shape[1] || l.dtype != r.dtype)
        die("oracle: invalid matmul dimensions");
    size_t b = l.shape[0], m = l.shape[1], k = l.shape[2], n = r.shape[2];
    Tensor out = Tensor::make(l.dtype, {b, m, n});
    if (l.dtype == F32) {
        for (size_t i = 0; i < b; i++) gemm_acc<float>(l.ptr<float>() + i * m * k, r.ptr<float>() + i * k * n, out.ptr<float>() + i * m * n, m, k, n);
    } else if (l.dtype == F64) {
        for (size_t i = 0; i < b; i++) gemm_acc<double>(l.ptr<double>() + i * m * k, r.ptr<double>() + i * k * n, out.ptr<double>() + i * m * n, m, k, n);
    } else if (l.dtype == F16) {
        // f16 storage, f32 accumulation, one rounding at the end
        std::vector<float> a(b * m * k), bb(b * k * n), c(b * m * n, 0.0f);
        for (size_t i = 0; i < a.size(); i++) a[i] = h2f(l.ptr<uint16_t>()[i]);
        for (size_t i = 0; i < bb.size(); i++) bb[i] = h2f(r.ptr<uint16_t>()[i]);
        for (size_t i = 0; i < b; i++) gemm_acc<float>(a.data() + i * m * k, bb.data() + i * k * n, c.data() + i * m * n, m, k, n);
        for (size_t i = 0; i < c.size(); i++) out.ptr<uint16_t>()[i] = f2h(c[i]);
    } else {
        dispatch(l.dtype, [&](auto *tp) {
            using T = std::remove_pointer_t<decltype(tp)>;
            if constexpr (std::is_integral<T>::value && !std::is_same<T, bool>::value) {
                using U = std::make_unsigned_t<T>;
                for (size_t i = 0; i < b; i++) gemm_acc<U>((const U *) l.ptr<T>() + i * m * k, (const U *) r.ptr<T>() + i * k * n, (U *) out.ptr<T>() + i * m * n, m, k, n);
            } else {
                die("oracle: matmul on this dtype is not supported");
            }
            return 0;
        });
    }
    return out;
}

Tensor eval_conv(const Node &nd, const Tensor &input, const Tensor &filter) {
    // cpu.rs:347-419: im2col, then one matrix product, then back to NCHW
    if (input.dtype != F32 || filter.dtype != F32) die("oracle: conv is only restated for f32");
    size_t sy = nd.conv[0], sx = nd.conv[1], py = nd.conv[2], px = nd.conv[3], kh = nd.conv[4], kw = nd.conv[5], oh = nd.conv[6], ow = nd.conv[7];
    size_t batch = input.shape[0], ic = input.shape[1], ih = input.shape[2], iw = input.shape[3], oc = filter.shape[0];
    size_t rows = batch * oh * ow, K = ic * kh * kw;
    std::vector<float> col(rows * K, 0.0f);
    const float *in = input.ptr<float>();
    for (size_t b = 0; b < batch; b++)
        for (size_t oy = 0; oy < oh; oy++)
            for (size_t ox = 0; ox < ow; ox++) {
                float *row = col.data() + ((b * oh + oy) * ow + ox) * K;
                for (size_t c = 0; c < ic; c++)
                    for (size_t fy = 0; fy < kh; fy++)
                        for (size_t fx = 0; fx < kw; fx++) {
                            int64_t iy = (int64_t) (oy * sy + fy) - (int64_t) py, ix = (int64_t) (ox * sx + fx) - (int64_t) px;
                            if (iy >= 0 && iy < (int64_t) ih && ix >= 0 && ix < (int64_t) iw)
                                row[(c * kh + fy) * kw + fx] = in[((b * ic + c) * ih + iy) * iw + ix];
                        }
            }
    // kernel matrix [K, oc]
    std::vector<float> km(K * oc);
    const float *f = filter.ptr<float>();
    for (size_t o = 0; o < oc; o++)
        for (size_t k = 0; k < K; k++) km[k * oc + o] = f[o * K + k];
    std::vector<float> res(rows * oc, 0.0f);
    gemm_acc<float>(col.data(), km.data(), res.data(), rows, K, oc);
    Tensor out = Tensor::make(F32, {batch, oc, oh, ow});
    float *op = out.ptr<float>();
    for (size_t b = 0; b < batch; b++)
        for (size_t p = 0; p < oh * ow; p++)
            for (size_t o = 0; o < oc; o++) op[(b * oc + o) * oh * ow + p] = res[(b * oh * ow + p) * oc + o];
    return out;
}

// view the tensor as [outer, len, inner] around `axis`
void split_axis(const std::vector<size_t> &shape, size_t axis, size_t *outer, size_t *len, size_t *inner) {
    *outer = 1;
    *inner = 1;
    for (size_t a = 0; a < axis; a++) *outer *= shape[a];
    *len = shape[axis];
    for (size_t a = axis + 1; a < shape.size(); a++) *inner *= shape[a];
}

float rust_max(float a, float b) { return std::isnan(a) ? b : (std::isnan(b) ? a : (a > b ? a : b)); }

// F16 tensors (absent from the reference) as f32 and back: row operations load f16, compute in f32 and round once.
Tensor widen_f16(const Tensor &x) {
    Tensor out = Tensor::make(F32, x.shape);
    size_t n = out.len();
    for (size_t i = 0; i < n; i++) out.ptr<float>()[i] = h2f(x.ptr<uint16_t>()[i]);
    return out;
}

Tensor narrow_f16(const Tensor &x) {
    Tensor out = Tensor::make(F16, x.shape);
    size_t n = x.len();
    for (size_t i = 0; i < n; i++) out.ptr<uint16_t>()[i] = f2h(x.ptr<float>()[i]);
    return out;
}

Tensor eval_softmax(const Tensor &x, size_t axis) {
    // cpu.rs:443-458
    if (x.dtype == F16) return narrow_f16(eval_softmax(widen_f16(x), axis));
    if (x.dtype != F32) die("oracle: softmax input must be f32 or f16");
    Tensor out = Tensor::make(F32, x.shape);
    size_t outer, len, inner;
    split_axis(x.shape, axis, &outer, &len, &inner);
    const float *s = x.ptr<float>();
    float *d = out.ptr<float>();
    for (size_t o = 0; o < outer; o++)
        for (size_t i = 0; i < inner; i++) {
            const float *sp = s + o * len * inner + i;
            float *dp = d + o * len * inner + i;
            float mx = -INFINITY;
            for (size_t j = 0; j < len; j++) mx = rust_max(mx, sp[j * inner]);
            float sum = 0;
            for (size_t j = 0; j < len; j++) {
                float e = std::exp(sp[j * inner] - mx);
                dp[j * inner] = e;
                sum += e;
            }
            for (size_t j = 0; j < len; j++) dp[j * inner] /= sum;
        }
    return out;
}

Tensor eval_layernorm(const Tensor &x, size_t axis, float eps) {
    // cpu.rs:461-479: biased variance, eps inside the square root
    if (x.dtype == F16) return narrow_f16(eval_layernorm(widen_f16(x), axis, eps));
    if (x.dtype != F32) die("oracle: layernorm input must be f32 or f16");
    Tensor out = Tensor::make(F32, x.shape);
    size_t outer, len, inner;
    split_axis(x.shape, axis, &outer, &len, &inner);
    const float *s = x.ptr<float>();
    float *d = out.ptr<float>();
    for (size_t o = 0; o < outer; o++)
        for (size_t i = 0; i < inner; i++) {
            const float *sp = s + o * len * inner + i;
            float *dp = d + o * len * inner + i;
            float sum = 0;
            for (size_t j = 0; j < len; j++) sum += sp[j * inner];
            float mean = sum / (float) len;
            float sq = 0;
            for (size_t j = 0; j < len; j++) {
                float c = sp[j * inner] - mean;
                dp[j * inner] = c;
                sq += c * c;
            }
            float denom = std::sqrt(sq / (float) len + eps);
            for (size_t j = 0; j < len; j++) dp[j * inner] /= denom;
        }
    return out;
}

Tensor eval_reduce(const Node &nd, const Tensor &x, const std::vector<size_t> &out_shape) {
    // cpu.rs:259-272 with graph.rs:1746-1786: one axis at a time, each lane folded left to right from the identity
    Tensor curr = x;
    for (size_t axis : nd.axes) {
        std::vector<size_t> ns = curr.shape;
        ns[axis] = 1;
        Tensor next = Tensor::make(curr.dtype, ns);
        size_t outer, len, inner;
        split_axis(curr.shape, axis, &outer, &len, &inner);
        auto run = [&](auto *tp, auto identity_of, auto from, auto to) {
            using T = std::remove_pointer_t<decltype(tp)>;
            uint8_t bop = nd.sub == Prod ? Mul : nd.sub == RMin ? Min : nd.sub == RMax ? Max : Add;
            for (size_t o = 0; o < outer; o++)
                for (size_t i = 0; i < inner; i++) {
                    T acc = identity_of();
                    for (size_t j = 0; j < len; j++) acc = binary_scalar<T>(bop, acc, from(o * len * inner + j * inner + i));
                    if (nd.sub == Mean) {
                        if constexpr (std::is_same<T, float>::value) acc = acc / (float) len;
                    }
                    to(o * inner + i, acc);
                }
        };
        if (curr.dtype == F16) {
            const uint16_t *s = curr.ptr<uint16_t>();
            uint16_t *d = next.ptr<uint16_t>();
            // f32 accumulation over the lane, one rounding at the end
            float ident = nd.sub == Prod ? 1.0f : nd.sub == RMin ? INFINITY : nd.sub == RMax ? -INFINITY : 0.0f;
            uint8_t bop = nd.sub == Prod ? Mul : nd.sub == RMin ? Min : nd.sub == RMax ? Max : Add;
            for (size_t o = 0; o < outer; o++)
                for (size_t i = 0; i < inner; i++) {
                    float acc = ident;
                    for (size_t j = 0; j < len; j++) acc = binary_scalar<float>(bop, acc, h2f(s[o * len * inner + j * inner + i]));
                    if (nd.sub == Mean) acc = acc / (float) len;
                    d[o * inner + i] = f2h(acc);
                }
        } else {
            dispatch(curr.dtype, [&](auto *tp) {
                using T = std::remove_pointer_t<decltype(tp)>;
                if constexpr (!std::is_same<T, half_t>::value) {
                    const T *s = curr.ptr<T>();
                    T *d = next.ptr<T>();
                    auto identity_of = [&]() -> T {
                        if constexpr (std::is_same<T, bool>::value) return nd.sub == Prod || nd.sub == RMin;
                        else if constexpr (std::is_floating_point<T>::value)
                            return nd.sub == Prod ? (T) 1 : nd.sub == RMin ? (T) INFINITY : nd.sub == RMax ? (T) -INFINITY : (T) 0;
                        else
                            return nd.sub == Prod ? (T) 1 : nd.sub == RMin ? std::numeric_limits<T>::max()
                                   : nd.sub == RMax ? std::numeric_limits<T>::min() : (T) 0;
                    };
                    run(tp, identity_of, [&](size_t k) { return s[k]; }, [&](size_t k, T v) { d[k] = v; });
                }
                return 0;
            });
        }
        curr = next;
    }
    curr.shape = out_shape;
    return curr;
}

Tensor eval_gather(const Tensor &x, size_t axis, const Tensor &indices, const std::vector<size_t> &out_shape) {
    // cpu.rs:304-333: negative or out of range indices are errors
    if (indices.shape.size() != 1) die("oracle: gather indices must have rank 1");
    Tensor out = Tensor::make(x.dtype, out_shape);
    size_t outer, len, inner;
    split_axis(x.shape, axis, &outer, &len, &inner);
    size_t n = indices.len(), es = dt_bytes(x.dtype);
    std::vector<size_t> idx(n);
    dispatch(indices.dtype, [&](auto *tp) {
        using T = std::remove_pointer_t<decltype(tp)>;
        if constexpr (std::is_integral<T>::value && !std::is_same<T, bool>::value) {
            for (size_t j = 0; j < n; j++) {
                T v = indices.ptr<T>()[j];
                if constexpr (std::is_signed<T>::value) {
                    if (v < 0) die("oracle: negative gather index");
                }
                if ((uint64_t) v >= len) die("oracle: Index out of bounds");
                idx[j] = (size_t) v;
            }
        } else {
            die("oracle: gather indices should be integers");
        }
        return 0;
    });
    for (size_t o = 0; o < outer; o++)
        for (size_t j = 0; j < n; j++)
            memcpy(out.data->data() + ((o * n + j) * inner) * es, x.data->data() + ((o * len + idx[j]) * inner) * es, inner * es);
    return out;
}

struct Result {
    std::vector<Tensor> outputs;
};

thread_local std::string g_error;

Result *run(const uint8_t *blob, size_t len, uint64_t batch, const void *const *inputs, size_t n_inputs) {
    ParsedGraph g = parse(blob, len);
    if (n_inputs != g.inputs.size()) die("oracle: Wrong input count");
    size_t n = g.nodes.size();
    // last use of every value, so that big intermediates are dropped early (cpu.rs:60-76)
    std::vector<size_t> last_use(n, 0);
    for (size_t i = 0; i < n; i++)
        for (uint32_t in : g.nodes[i].inputs) last_use[in] = i;
    for (uint32_t o : g.outputs) last_use[o] = n;
    std::vector<Tensor> vals(n);
    for (size_t i = 0; i < n; i++) {
        const Node &nd = g.nodes[i];
        std::vector<size_t> out_shape;
        for (auto &s : nd.shape) out_shape.push_back(s.eval(batch));
        auto in = [&](size_t k) -> const Tensor & {
            const Tensor &t = vals[nd.inputs[k]];
            if (!t.data) die("oracle: operand was freed too early");
            return t;
        };
        Tensor result;
        switch (nd.op) {
            case Input: {
                result = Tensor::make(nd.dtype, out_shape);
                if (result.data->size()) memcpy(result.data->data(), inputs[nd.index], result.data->size());
                break;
            }
            case Constant: result = nd.constant; break;
            case View:
                result = in(0);
                result.shape = out_shape;
                break;
            case Broadcast: {
                const Tensor &x = in(0);
                auto st = dense_strides(x.shape);
                for (size_t a = 0; a < st.size(); a++)
                    if (x.shape[a] != out_shape[a]) st[a] = 0;
                result = gather_strided(x, out_shape, st, 0);
                break;
            }
            case Permute: {
                const Tensor &x = in(0);
                auto st = dense_strides(x.shape);
                std::vector<int64_t> ps;
                for (size_t a : nd.axes) ps.push_back(st[a]);
                result = gather_strided(x, out_shape, ps, 0);
                break;
            }
            case Slice: {
                const Tensor &x = in(0);
                auto st = dense_strides(x.shape);
                size_t a = nd.axes[0];
                int64_t off = st[a] * (int64_t) nd.start;
                st[a] *= (int64_t) nd.step;
                bool empty = false;
                for (size_t d : out_shape) empty |= d == 0;
                result = gather_strided(x, out_shape, st, empty ? 0 : off);
                break;
            }
            case Flip: {
                const Tensor &x = in(0);
                auto st = dense_strides(x.shape);
                size_t a = nd.axes[0];
                int64_t off = x.len() ? st[a] * (int64_t) (x.shape[a] - 1) : 0;
                st[a] = -st[a];
                result = gather_strided(x, out_shape, st, off);
                break;
            }
            case Gather: result = eval_gather(in(0), nd.axes[0], in(1), out_shape); break;
            case Concat: {
                result = Tensor::make(nd.dtype, out_shape);
                size_t axis = nd.axes[0], outer, len_o, inner, es = dt_bytes(nd.dtype), start = 0;
                split_axis(out_shape, axis, &outer, &len_o, &inner);
                for (size_t k = 0; k < nd.inputs.size(); k++) {
                    const Tensor &x = in(k);
                    size_t l = x.shape[axis];
                    for (size_t o = 0; o < outer; o++)
                        memcpy(result.data->data() + ((o * len_o + start) * inner) * es, x.data->data() + (o * l * inner) * es, l * inner * es);
                    start += l;
                }
                if (start != len_o) die("oracle: concat sizes do not add up");
                break;
            }
            case Conv: result = eval_conv(nd, in(0), in(1)); break;
            case MatMul: result = eval_matmul(in(0), in(1)); break;
            case Unary: result = eval_unary(nd, in(0), out_shape); break;
            case Binary: result = eval_binary(nd, in(0), in(1)); break;
            case Softmax: result = eval_softmax(in(0), nd.axes[0]); break;
            case Layernorm: result = eval_layernorm(in(0), nd.axes[0], nd.eps); break;
            case Reduce: result = eval_reduce(nd, in(0), out_shape); break;
        }
        if (result.shape != out_shape) die("oracle: Wrong output shape");
        if (result.dtype != nd.dtype) die("oracle: Wrong output dtype");
        vals[i] = std::move(result);
        for (uint32_t inp : nd.inputs)
            if (last_use[inp] == i) vals[inp] = Tensor();
        if (last_use[i] == 0) vals[i] = Tensor();  // never used and not an output
    }
    Result *res = new Result();
    for (uint32_t o : g.outputs) res->outputs.push_back(vals[o]);
    return res;
}

}  // namespace

extern "C" {

const char *kn_oracle_last_error(void) { return g_error.c_str(); }

// inputs: dense row-major buffers in graph input order, shaped as the graph's input shapes at `batch`
int kn_oracle_eval(const uint8_t *blob, size_t len, uint64_t batch, const void *const *inputs, size_t n_inputs, void **handle) {
    try {
        *handle = run(blob, len, batch, inputs, n_inputs);
        return 0;
    } catch (const std::exception &e) {
        g_error = e.what();
        return 1;
    }
}

size_t kn_oracle_output_count(void *handle) { return ((Result *) handle)->outputs.size(); }

// dims needs room for `cap` entries
int kn_oracle_output_info(void *handle, size_t i, int *dtype, size_t *rank, size_t *dims, size_t cap, const void **data, size_t *bytes) {
    Result *r = (Result *) handle;
    if (i >= r->outputs.size()) return 1;
    const Tensor &t = r->outputs[i];
    *dtype = t.dtype;
    *rank = t.shape.size();
    if (cap < t.shape.size()) return 2;
    for (size_t k = 0; k < t.shape.size(); k++) dims[k] = t.shape[k];
    *data = t.data->data();
    *bytes = t.data->size();
    return 0;
}

void kn_oracle_free(void *handle) { delete (Result *) handle; }

}  // extern "C"
