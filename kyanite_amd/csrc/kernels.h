// Generators for the run-time compiled gfx950 kernels ("autokernels"): fused elementwise chains / strided copy,
// reduce, softmax, layernorm and gather. They take the role of kn-cuda-eval/src/autokernel/{scalar,reduce,softmax,
// layernorm,gather}.rs + the matching .cu templates, but the device code is new and written for CDNA4:
// wave64 shuffles, 128-bit accesses on the contiguous axis, rows held in registers so HBM is touched once per
// element, and all index arithmetic against compile-time constants.
#pragma once

#include "strided_shape.h"

namespace kn {

// Choices of the generators that a caller may move; the generators of a thread read the options of the innermost
// GeneratorScope alive on it (the defaults when there is none).
struct GeneratorOptions {
    // operands of at least this many bytes that are touched once per element are read and written with non-temporal
    // accesses (0: never)
    size_t streaming_bytes = (size_t) 64 << 20;
    // elementwise kernels with an operand that is contiguous along another axis than the outputs turn 64 x 64 tiles
    // through LDS (off: the plain kernel with strided accesses)
    bool tiled_transpose = true;
};
class GeneratorScope {
public:
    explicit GeneratorScope(const GeneratorOptions &options);
    ~GeneratorScope();
    GeneratorScope(const GeneratorScope &) = delete;
    GeneratorScope &operator=(const GeneratorScope &) = delete;

private:
    const GeneratorOptions *previous_;
    GeneratorOptions mine_;
};
const GeneratorOptions &generator_options();

// A kernel ready to be compiled: every shape, stride and expression is baked into `source`; the only launch
// arguments are the operand base addresses, in `operands` order.
struct KernelSpec {
    std::string name;    // entry point
    std::string source;  // complete translation unit
    uint32_t grid = 0;   // number of workgroups; 0 means nothing to do
    uint32_t block = 0;  // threads per workgroup
    size_t n_ptrs = 0;
    std::string strategy;  // human readable note on the specialisation that was picked
    // Row kernels only: whether the rows are held in registers (read once), or read again per pass by the one workgroup
    // that owns a row (lanes along the row) or a few columns (lanes across neighbouring columns)
    enum RowAccess { RowsHeld, RowsStreamed, ColumnsStreamed } row_access = RowsHeld;
};

// One node of a fused elementwise expression: operands are loaded (`Load`), single-valued constants are inlined
// (`Const`), everything else refers to earlier nodes.
// `Raw`: statements in the form the reference writes its operations in, "*x0 = *x1 + *x2;" (autokernel/scalar.rs:36):
// x0 points at the result, xk at the loaded operand k, each in its register type (f16 as float, bool as bool).
// A Raw node is the last node of its expression and follows one Load node per operand it may read.
struct ScalarNode {
    enum Kind { Load, Const, Unary, Binary, Raw } kind = Load;
    DType dtype = DType::F32;  // type of the produced value
    size_t operand = 0;        // Load: index into the operand list
    DScalar constant;          // Const
    UnaryOp unary = UnaryOp::Abs;
    DType cast_to = DType::F32;
    BinaryOp binary = BinaryOp::Add;
    size_t a = 0, b = 0;  // argument node indices
    std::string raw;      // Raw: the statements
};

// An expression DAG in evaluation order, the last node being the result.
struct ScalarExpr {
    std::vector<ScalarNode> nodes;
    size_t result() const { return nodes.size() - 1; }
};

struct KernelOperand {
    DType dtype;
    StridedShape shape;
    int64_t offset_bytes;  // offset of the view origin inside its buffer, known at plan time (for alignment)
};

// out = expr(loads...). operands[0] is the output; the rest are the loaded operands, all of the same shape.
KernelSpec make_scalar_kernel(const std::vector<KernelOperand> &operands, const ScalarExpr &expr);
// Several results from one pass: operands[0 .. exprs.size()) are the outputs, one expression each, the rest are the
// loaded operands that all expressions share (Load nodes index the whole operand list).
KernelSpec make_scalar_kernel_multi(const std::vector<KernelOperand> &operands, const std::vector<ScalarExpr> &exprs);

// output[kept] = post(fold(op, pre(input[kept, reduced...]))) (reduce.rs:35-153). `pre`: an optional elementwise
// expression of the loaded element (its only operand is number 1), e.g. the square in a mean of squares.
// A reduction with few results and a long reduced index has too few workgroups to pull the input at the rate of the
// memory. With `split` given, such a reduction comes back as two kernels: the returned one folds `parts` slices of
// the reduced index side by side into partial[parts][kept] (elements of `partial_dtype`, the type the fold computes
// in; its second pointer is that array instead of the output), and `final` (pointers: partial, output) folds the
// slices in order and applies the mean's division. `parts` stays 1 when there is nothing to gain.
struct ReduceSplit {
    size_t parts = 1;
    size_t kept_size = 0;
    DType partial_dtype = DType::F32;
    size_t partial_words = 1;  // elements of `partial_dtype` per partial result (more than one for a ReduceStat)
    KernelSpec final;
};
// The statistics of a softmax or a layernorm as a reduction of its own, for rows (or columns) that no workgroup can
// hold: instead of one value per kept element the kernel folds a pair and stores TWO floats, one at its place in
// `output` and one `plane` floats behind that (two planes of the kept shape, one after the other):
//   MaxSumExp: the maximum m of the row and 1 / sum(exp(x - m)), the sum kept relative to the running maximum;
//   MeanRstd:  the mean and 1 / sqrt(variance + eps), from (count, mean, M2) triples (Welford per element, combined
//              pairwise after Chan, Golub and LeVeque).
// `op` is ignored then; -inf, +inf and NaN elements give what exp(x - max) / sum gives element by element.
struct ReduceStat {
    enum Kind { MaxSumExp, MeanRstd } kind = MaxSumExp;
    float eps = 0;
    size_t plane = 0;
};
KernelSpec make_reduce_kernel(const KernelOperand &input, const KernelOperand &output, const std::vector<size_t> &axes,
                              ReduceOp op, const ScalarExpr *pre = nullptr, ReduceSplit *split = nullptr,
                              const ReduceStat *stat = nullptr);

// Row kernels. The value that gets normalised is `pre(load operands...)`, the value stored is
// `post(normalised, load operands...)`: this is how a preceding scale / residual add and a following affine
// (gamma, beta) or activation are fused into the single pass over the row.
// Kind Reduce: the row statistic `fold(reduce_op, pre(...))` takes the place of the normalised value, the same for
// every element of the row (an RMS norm: pre = x * x, mean, post = x * rsqrt(stat + eps) * w).
struct RowKernelDesc {
    enum Kind { Softmax, Layernorm, Reduce } kind = Softmax;
    ReduceOp reduce_op = ReduceOp::Sum;  // Sum, Mean, Max or Min
    size_t axis = 0;
    float eps = 0;
    // operands[0] is the output, operands[1..] are inputs; every operand has the full (output) shape
    std::vector<KernelOperand> operands;
    ScalarExpr pre;   // over Load nodes only; result f32
    ScalarExpr post;  // Load nodes refer to operands; the node with kind Load and operand == SIZE_MAX is the normalised value
};
KernelSpec make_row_kernel(const RowKernelDesc &desc);

// output[kept.., i, kept..] = input[kept.., indices[i], kept..], zero when the index is out of range (gather.rs:30-129)
KernelSpec make_gather_kernel(const KernelOperand &input, const KernelOperand &indices, const KernelOperand &output,
                              size_t axis);

// Common device-side helpers prepended to every generated kernel.
const char *kernel_prelude();

}  // namespace kn
