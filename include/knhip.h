/* knhip.h - C ABI of libknhip, the MI355X (gfx950) executor for Kyanite graphs.
 *
 * This is what a `kn-hip-sys` crate binds in place of `kn-cuda-sys`. Every function returns 0 on success and a
 * non-zero status otherwise; `knhip_last_error()` then describes the failure (thread local). No exception or
 * panic crosses this boundary: where the reference panics (kn-cuda-sys/src/wrapper/status.rs:9-33 and the asserts
 * of kn-cuda-eval/src/executor.rs:118-127) these functions report an error, and a binding can turn it back into
 * a panic to keep the reference's behaviour.
 *
 * Handles are not thread safe (the reference's executor is Send but takes &mut self, executor.rs:41, :117);
 * every entry point selects its device itself (handle.rs:60-64).
 *
 * File/line citations name the reference interface each group replaces, relative to the Kyanite repository.
 */
#ifndef KNHIP_H
#define KNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status ------------------------------------------------------------------------------------------------ */
#define KNHIP_OK 0
#define KNHIP_ERROR 1          /* contract violation or runtime failure, see knhip_last_error() */
#define KNHIP_BUFFER_TOO_SMALL 2

const char *knhip_last_error(void);

/* ---- element types (kn-graph/src/dtype.rs:24-37, plus F16) --------------------------------------------------- */
enum {
    KNHIP_F32 = 0, KNHIP_F64 = 1, KNHIP_I8 = 2, KNHIP_I16 = 3, KNHIP_I32 = 4, KNHIP_I64 = 5,
    KNHIP_U8 = 6, KNHIP_U16 = 7, KNHIP_U32 = 8, KNHIP_U64 = 9, KNHIP_BOOL = 10, KNHIP_F16 = 11
};

/* one dimension `fixed_factor * batch_size^batch_exp` (kn-graph/src/shape.rs:31-38) */
typedef struct {
    uint64_t fixed_factor;
    uint32_t batch_exp;
} knhip_size_t;

/* operation codes as stored in value infos and in the serialised graph (kn-graph/src/graph.rs:106-162) */
enum {
    KNHIP_OP_INPUT = 0, KNHIP_OP_CONSTANT = 1, KNHIP_OP_VIEW = 2, KNHIP_OP_BROADCAST = 3, KNHIP_OP_PERMUTE = 4,
    KNHIP_OP_SLICE = 5, KNHIP_OP_FLIP = 6, KNHIP_OP_GATHER = 7, KNHIP_OP_CONCAT = 8, KNHIP_OP_CONV = 9,
    KNHIP_OP_MATMUL = 10, KNHIP_OP_UNARY = 11, KNHIP_OP_BINARY = 12, KNHIP_OP_SOFTMAX = 13, KNHIP_OP_LAYERNORM = 14,
    KNHIP_OP_REDUCE = 15
};
/* graph.rs:173-195 */
enum {
    KNHIP_UNARY_ABS = 0, KNHIP_UNARY_NEG = 1, KNHIP_UNARY_SIN = 2, KNHIP_UNARY_COS = 3, KNHIP_UNARY_EXP = 4,
    KNHIP_UNARY_LOG = 5, KNHIP_UNARY_SQRT = 6, KNHIP_UNARY_SIGMOID = 7, KNHIP_UNARY_TANH = 8, KNHIP_UNARY_ERF = 9,
    KNHIP_UNARY_MISH = 10, KNHIP_UNARY_SOFTPLUS = 11, KNHIP_UNARY_VALUE_CAST = 12, KNHIP_UNARY_BIT_CAST = 13
};
/* graph.rs:197-206 */
enum { KNHIP_BINARY_ADD = 0, KNHIP_BINARY_SUB = 1, KNHIP_BINARY_MUL = 2, KNHIP_BINARY_DIV = 3, KNHIP_BINARY_MIN = 4,
       KNHIP_BINARY_MAX = 5, KNHIP_BINARY_POW = 6 };
/* graph.rs:208-217 */
enum { KNHIP_REDUCE_SUM = 0, KNHIP_REDUCE_MEAN = 1, KNHIP_REDUCE_PROD = 2, KNHIP_REDUCE_MAX = 3, KNHIP_REDUCE_MIN = 4 };

/* ---- device and memory shim (replaces kn-cuda-sys/src/wrapper/handle.rs:37-103 and mem/{device,pinned}.rs) ---- */
int knhip_device_count(int *count);
int knhip_device_name(int device, char *buf, size_t cap, size_t *needed);
int knhip_malloc(int device, size_t bytes, void **ptr);
int knhip_free(int device, void *ptr);
int knhip_memcpy_h2d(int device, void *dst, const void *src, size_t bytes);
int knhip_memcpy_d2h(int device, void *dst, const void *src, size_t bytes);
int knhip_memcpy_d2d(int device, void *dst, const void *src, size_t bytes);
int knhip_host_alloc(size_t bytes, void **ptr);
int knhip_host_free(void *ptr);
int knhip_device_synchronize(int device);

/* streams and events (replaces CudaStream, kn-cuda-sys/src/wrapper/handle.rs:105-174, and CudaEvent, event.rs:7-45).
 * Handles are the HIP objects themselves (hipStream_t / hipEvent_t behind void *); a NULL stream is the device's
 * default stream. Every stream has the default priority. An event belongs to the device it was created on. */
int knhip_stream_create(int device, void **stream);                      /* CudaStream::new, handle.rs:124-131 */
int knhip_stream_destroy(int device, void *stream);                      /* Drop, handle.rs:115-121 */
int knhip_stream_synchronize(int device, void *stream);                  /* handle.rs:133-135 */
int knhip_stream_wait_event(int device, void *stream, void *event);      /* wait_for_event, handle.rs:155-159 */
int knhip_event_create(int device, void **event);                        /* CudaEvent::new, event.rs:10-16 */
int knhip_event_destroy(int device, void *event);                        /* Drop, event.rs:40-44 */
int knhip_event_record(int device, void *event, void *stream);           /* record_existing_event, handle.rs:151-153 */
int knhip_event_synchronize(int device, void *event);                    /* event.rs:28-30 */
/* seconds between two recorded events, like CudaEvent::time_elapsed_since (event.rs:19-26) */
int knhip_event_elapsed_seconds(int device, void *start, void *end, float *seconds);
/* copies that return once queued on `stream` (copy_linear_{from,to}_host_async, mem/device.rs:114-153): the host
 * side must be pinned memory (knhip_host_alloc) that stays untouched until the stream has passed the copy */
int knhip_memcpy_h2d_async(int device, void *dst, const void *src, size_t bytes, void *stream);
int knhip_memcpy_d2h_async(int device, void *dst, const void *src, size_t bytes, void *stream);
int knhip_memcpy_d2d_async(int device, void *dst, const void *src, size_t bytes, void *stream);

/* ---- one batched matrix product on device memory, outside any executor ---------------------------------------
 * The role of BatchedMatMulArgs::run (kn-cuda-sys/src/wrapper/group.rs:107-171, cublasSgemm[StridedBatched]):
 * C[b] = A[b] B[b] for b < batch, A [m, k], B [k, n], C [m, n], every matrix addressed by element strides (batch, row,
 * column; a zero batch stride broadcasts the matrix). cuBLAS operands map onto this directly: a column-major operand
 * with leading dimension ld has row stride 1 and column stride ld, a transposed one the other way round, and
 * MatMulOperand::stride is the batch stride. alpha = 1 and beta = 0, the only values the reference passes
 * (kn-cuda-eval/src/planner.rs:606-648). Elements are f32, or f16 with f32 accumulation and one rounding at the store.
 * Launches that split the K axis between workgroups keep f32 partial products and tile counters in `workspace`
 * (device memory, 256 byte aligned, knhip_batched_mat_mul_workspace_bytes(args) bytes; may be NULL when that is 0);
 * the call returns once the work is queued on `stream`, and the workspace must stay untouched until it has run.
 * A batch of more than 65535 entries runs as several launches, one after the other on `stream`. */
typedef struct {
    int dtype; /* KNHIP_F32 or KNHIP_F16 */
    int batch, m, n, k;
    const void *a;
    int64_t a_batch_stride, a_row_stride, a_col_stride;
    const void *b;
    int64_t b_batch_stride, b_row_stride, b_col_stride;
    void *c;
    int64_t c_batch_stride, c_row_stride, c_col_stride;
} knhip_matmul_args;
int knhip_batched_mat_mul_workspace_bytes(const knhip_matmul_args *args, size_t *bytes);
int knhip_batched_mat_mul(int device, void *stream, const knhip_matmul_args *args, void *workspace, size_t workspace_bytes);

/* No counterpart in the reference. For callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): knhip_batched_mat_mul with the workspace taken from a static
 * device array of KNHIP_STATIC_SCRATCH_BYTES per GPU instead of an argument. The call allocates nothing and fails
 * with a message when the product needs more scratch than that. All calls on one GPU share the array: calls whose
 * work overlaps on one GPU (two streams, two threads) race, the caller orders them. */
#define KNHIP_STATIC_SCRATCH_BYTES (32u << 20)
int knhip_batched_mat_mul_static(int device, void *stream, const knhip_matmul_args *args);
/* The first use of the static array on a device looks its address up, which is no stream operation and may be refused
 * while a stream capture is open: call this once per device beforehand (any earlier knhip_batched_mat_mul_static on the
 * device does the same). Allocates nothing. */
int knhip_static_scratch_prepare(int device);

/* ---- device tensors and stand-alone kernels, outside any executor ------------------------------------------------
 * A tensor in device memory that the caller owns: DeviceTensor = PtrTensor<DevicePtr> (kn-cuda-eval/src/
 * offset_tensor.rs:14-20, device_tensor.rs:12). `ptr` is the address of the element with index 0 along every axis,
 * strides are in elements and may be zero (broadcast) or negative (flipped); the views of offset_tensor.rs:52-114
 * (permute, view, broadcast, slice, index, flip, repeat_unary) are edits of shape, strides and address that the
 * binding does on its side (knhip_strided_view / knhip_strided_slice below give the layout algebra). */
typedef struct {
    void *ptr;
    int dtype; /* KNHIP_F32 ... KNHIP_F16 */
    size_t rank;
    const size_t *shape;
    const int64_t *strides;
} knhip_tensor;

/* DeviceTensor::copy_from (device_tensor.rs:101-126): dst[i] = src[i] for every index i of the common shape, same
 * dtype. One linear device-to-device copy when both sides have the same dense strides, else the elementwise kernel
 * with the operation `y = x` on the two layouts (the reference's "restride trick", copy_from_as_scalar_op
 * :73-99). Returns once the work is queued on `stream` (the reference synchronises a stream of its own; a binding that
 * wants that calls knhip_stream_synchronize). The destination may not have a broadcast axis. */
int knhip_strided_copy(int device, void *stream, const knhip_tensor *dst, const knhip_tensor *src);

/* The five run-time compiled kernel types of kn-cuda-eval/src/autokernel/, on caller-owned tensors. A constructor
 * specialises the kernel for shapes, strides and element types (tensor descriptors whose `ptr` may be NULL: the tensor
 * is then assumed to start on a 16 byte boundary; run refuses addresses of another alignment than the constructor
 * saw) and compiles it (cached). `device` -1 compiles without a GPU; such a kernel cannot run. knhip_kernel_run takes
 * the addresses in the order of the constructor's tensors and returns once the launch is queued on `stream`. */
typedef struct knhip_kernel knhip_kernel;
/* ScalarKernel::new_for_shapes (autokernel/scalar.rs:33-121): `operation` in the reference's form, "*x0 = *x1 + *x2;"
 * (it must end in ';'). x0 points at the element of operand 0, which is written; xk (k >= 1) at the element of
 * operand k, which is read. Inside the operation a value has its register type: float for f16, bool for bool, else the
 * C type of its dtype. All operands have one shape; run: one address per operand. */
int knhip_scalar_kernel_new(int device, const char *operation, const knhip_tensor *operands, size_t operand_count,
                            knhip_kernel **out);
/* ReduceKernel::new (autokernel/reduce.rs:35-123) with the operation as a code (KNHIP_REDUCE_*, identities and mean
 * as in kn-graph/src/graph.rs:1746-1786) where the reference takes C text; `output` has the kept axes of `input` in
 * order. run: (input, output). */
int knhip_reduce_kernel_new(int device, int reduce_op, const knhip_tensor *input, const knhip_tensor *output, const size_t *axes,
                            size_t axis_count, knhip_kernel **out);
/* SoftmaxKernel::new (autokernel/softmax.rs:28-91): output = softmax(input_scale * input) along `axis`, f32.
 * run: (input, output). */
int knhip_softmax_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *output, size_t axis, float input_scale,
                             knhip_kernel **out);
/* LayernormKernel::new (autokernel/layernorm.rs:33-93): x = alpha0 * input0 + alpha1 * input1, output =
 * beta * (x - mean) / sqrt(var + eps) along `axis`, f32; input1 has input0's layout and is only read when alpha1 is
 * not 0. run: (input0, input1 or NULL, output), like layernorm.rs:95-111. */
int knhip_layernorm_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *output, size_t axis, float eps,
                               float alpha0, float alpha1, float beta, knhip_kernel **out);
/* GatherKernel::new (autokernel/gather.rs:30-98): output[.., i, ..] = input[.., indices[i], ..] along `axis`, zero where
 * the index is out of range; indices of any integer type, rank 1. run: (input, indices, output). */
int knhip_gather_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *indices, const knhip_tensor *output,
                            size_t axis, knhip_kernel **out);
int knhip_kernel_run(const knhip_kernel *kernel, void *stream, void *const *ptrs, size_t count);
/* the specialisation that was picked (a short text), and the launch size */
int knhip_kernel_info(const knhip_kernel *kernel, char *strategy, size_t cap, size_t *needed, unsigned *grid, unsigned *block);
void knhip_kernel_free(knhip_kernel *kernel);

/* ---- graph (kn-graph/src/graph.rs) ------------------------------------------------------------------------- */
typedef struct knhip_graph knhip_graph;
typedef uint32_t knhip_value; /* index of a value inside its graph; values are append-only (graph.rs:86-91) */

int knhip_graph_new(knhip_graph **out);                                   /* graph.rs:364-373 */
int knhip_graph_clone(const knhip_graph *graph, knhip_graph **out);
void knhip_graph_free(knhip_graph *graph);
/* flat binary form, the way a host language hands over a graph built with its own kn-graph */
int knhip_graph_deserialize(const uint8_t *blob, size_t len, knhip_graph **out);
int knhip_graph_serialize(const knhip_graph *graph, uint8_t *buf, size_t cap, size_t *needed);
int knhip_graph_str(const knhip_graph *graph, char *buf, size_t cap, size_t *needed); /* graph.rs:1473-1512 */

/* builder, one entry per public builder method (graph.rs:583-1363) */
int knhip_graph_input(knhip_graph *g, const knhip_size_t *dims, size_t rank, int dtype, knhip_value *out);
int knhip_graph_constant(knhip_graph *g, const knhip_size_t *dims, size_t rank, int dtype, const void *data,
                         size_t data_bytes, knhip_value *out);
int knhip_graph_view(knhip_graph *g, knhip_value input, const knhip_size_t *dims, size_t rank, knhip_value *out);
int knhip_graph_broadcast(knhip_graph *g, knhip_value input, const knhip_size_t *dims, size_t rank, knhip_value *out);
int knhip_graph_repeat_unary(knhip_graph *g, knhip_value input, size_t axis, knhip_size_t count, knhip_value *out);
int knhip_graph_flatten(knhip_graph *g, knhip_value input, size_t start_axis, knhip_value *out);
int knhip_graph_permute(knhip_graph *g, knhip_value input, const size_t *permutation, size_t rank, knhip_value *out);
int knhip_graph_slice(knhip_graph *g, knhip_value input, size_t axis, size_t start, size_t end, size_t step,
                      knhip_value *out);
int knhip_graph_index(knhip_graph *g, knhip_value input, size_t axis, size_t index, knhip_value *out);
int knhip_graph_flip(knhip_graph *g, knhip_value input, size_t axis, knhip_value *out);
int knhip_graph_repeat(knhip_graph *g, knhip_value input, size_t axis, knhip_size_t count, int interleave,
                       knhip_value *out);
int knhip_graph_gather(knhip_graph *g, knhip_value input, size_t axis, knhip_value indices, knhip_value *out);
/* base_dims may be NULL (infer from the first input); dtype may be -1 (infer) */
int knhip_graph_concat(knhip_graph *g, const knhip_value *inputs, size_t count, size_t axis,
                       const knhip_size_t *base_dims, size_t base_rank, int dtype, knhip_value *out);
/* pad_amount holds rank (before, after) pairs */
int knhip_graph_pad(knhip_graph *g, knhip_value input, const size_t *pad_amount, size_t rank, knhip_value pad_value,
                    knhip_value *out);
int knhip_graph_conv(knhip_graph *g, knhip_value input, knhip_value filter, size_t stride_y, size_t stride_x,
                     size_t padding_y, size_t padding_x, knhip_value *out);
int knhip_graph_linear(knhip_graph *g, knhip_value input, knhip_value weight, knhip_value *out);
int knhip_graph_mat_mul(knhip_graph *g, knhip_value left, knhip_value right, knhip_value *out);
int knhip_graph_batched_mat_mul(knhip_graph *g, knhip_value left, knhip_value right, knhip_value *out);
int knhip_graph_softmax(knhip_graph *g, knhip_value input, size_t axis, knhip_value *out);
int knhip_graph_layernorm(knhip_graph *g, knhip_value input, size_t axis, float eps, knhip_value *out);
int knhip_graph_reduce(knhip_graph *g, knhip_value input, const size_t *axes, size_t count, int op, knhip_value *out);
/* min and max point at one element of the value's dtype */
int knhip_graph_clamp(knhip_graph *g, knhip_value input, const void *min, const void *max, knhip_value *out);
int knhip_graph_relu(knhip_graph *g, knhip_value input, knhip_value *out);
int knhip_graph_unary(knhip_graph *g, int op, int cast_dtype, knhip_value input, knhip_value *out);
int knhip_graph_binary(knhip_graph *g, int op, knhip_value left, knhip_value right, knhip_value *out);
/* graph.rs:1319-1351: inline `callee` into `g`; `outputs` receives callee's output count values */
int knhip_graph_call(knhip_graph *g, const knhip_graph *callee, const knhip_value *inputs, size_t input_count,
                     knhip_value *outputs, size_t output_cap, size_t *output_count);
int knhip_graph_output(knhip_graph *g, knhip_value value);
int knhip_graph_set_debug_id(knhip_graph *g, knhip_value value, const char *id);

/* queries */
int knhip_graph_value_count(const knhip_graph *g, size_t *count);
int knhip_graph_inputs(const knhip_graph *g, knhip_value *buf, size_t cap, size_t *count);
int knhip_graph_outputs(const knhip_graph *g, knhip_value *buf, size_t cap, size_t *count);
typedef struct {
    int dtype;
    int op;           /* KNHIP_OP_* */
    int sub_op;       /* unary / binary / reduce code, else -1 */
    int cast_dtype;   /* for casts, else -1 */
    size_t rank;
    size_t operand_count;
    size_t axis_count; /* permutation / axis / axes; for a conv: stride_y, stride_x, padding_y, padding_x */
    size_t non_output_uses;
    size_t slice_start, slice_end, slice_step;
    float eps;
    int is_hidden;
} knhip_value_info;
int knhip_graph_value_info(const knhip_graph *g, knhip_value value, knhip_value_info *info);
int knhip_graph_value_shape(const knhip_graph *g, knhip_value value, knhip_size_t *dims, size_t cap);
int knhip_graph_value_operands(const knhip_graph *g, knhip_value value, knhip_value *buf, size_t cap);
int knhip_graph_value_axes(const knhip_graph *g, knhip_value value, size_t *buf, size_t cap);
/* data of a Constant value: pointer stays valid as long as the graph lives */
int knhip_graph_value_constant(const knhip_graph *g, knhip_value value, const void **data, size_t *bytes);
/* graph.rs:490-527: 1 in *is_single and the element in `element` (8 bytes of room) when every element is equal */
int knhip_graph_as_single_const(const knhip_graph *g, knhip_value value, int *is_single, void *element);
/* Graph::as_const (graph.rs:435-474): the value computed on the host when it only depends on constants through
 * layout operations, unary / binary operations, reduce, gather and concat. *needed = byte size of the dense
 * row-major result (its shape and dtype are those of the value); the bytes are copied when cap >= *needed. */
int knhip_graph_as_const(const knhip_graph *g, knhip_value value, int *is_const, void *data, size_t cap, size_t *needed);

/* kn-graph/src/shape.rs:353-365. `actual` holds the concatenated dims of all inputs. *status: 0 ok, 1 different
 * length, 2 constant mismatch, 3 batch conflict, 4 impossible batch value; *has_batch 0 when any batch size fits */
int knhip_graph_infer_batch_size(const knhip_graph *g, const size_t *actual, const size_t *ranks, size_t input_count,
                                 int *status, int *has_batch, uint64_t *batch);

/* kn-graph/src/optimizer/mod.rs:11-46 */
typedef struct {
    int optimize;
    int force_bias_through_conv;
    int fuse_layernorm;
    int div_to_mul;
} knhip_optimizer_settings;
int knhip_optimizer_settings_default(knhip_optimizer_settings *settings);
int knhip_graph_optimize(const knhip_graph *g, const knhip_optimizer_settings *settings, knhip_graph **out);

/* ---- executor (kn-cuda-eval/src/executor.rs:60-258, kn-runtime/src/lib.rs:85-126) ------------------------------ */
typedef struct knhip_executor knhip_executor;

/* What an executor is built with beyond (device, graph, batch size). Fill the struct with
 * knhip_executor_options_default() and change what is needed; a NULL pointer means the defaults: the reference's
 * behaviour with every planned path of this library switched on. The options belong to the one executor (nothing is
 * read from the environment), so two executors of one process can be planned differently. The reference's own knob
 * surface is the optimizer's (kn-graph/src/optimizer/mod.rs:11-22, knhip_optimizer_settings above); its executor has
 * none (executor.rs:61).
 * plan_only: nothing touches a device, the graph is planned and its kernels are compiled (works on a machine without
 *   a GPU). preserve_inputs: input buffers are never reused for later values, for callers that write the inputs on the
 *   device once and then call run_async many times (the reference re-uploads them per evaluate). step_by_step: every
 *   run launches the planned steps one by one, also where the whole plan is small enough to run as one kernel
 *   (knhip_executor_fused_source).
 * The remaining int fields are 1 by default; 0 switches that path off:
 *   fuse_attention            matmul, softmax, matmul chains as one launch (off: three launches)
 *   fuse_gated_matmul         (x w_g) sigmoid(x w_g) (x w_u) in f16 as one launch whose store computes the gated
 *                             product (off: the two products, then an elementwise launch)
 *   group_matmuls             matmuls that share their left operand in one launch (off: one launch each)
 *   pack_matmul_constants     constant [k, n] right operands laid out again as [n, k] when the plan is made
 *   pointwise_conv_as_matmul  1 x 1 convolutions with stride 1 as one matrix product per image (off: the conv kernel)
 *   join_elementwise          neighbouring independent elementwise steps of one shape share a launch
 *   split_reduce              reductions with few results and a long reduced index run as two launches
 *   tiled_transpose           elementwise kernels with a transposed operand turn tiles through LDS
 *   split_conv_channels       convolutions with few tiles fold slices of their input channels side by side
 *   plane_conv_any_width      3 x 3 convolutions on images without a power-of-two width use the plane kernel
 *   direct_gemm               matmul kernels that load global -> LDS directly (off: staged through registers)
 *   split_k, tail_split       workgroups that share a tile along K (either kind) / only the last round's tiles
 *   dot_products              one wave per result for products of up to 2^20 multiplications
 * streaming_bytes: operands of at least this size that are touched once per element are read and written with
 *   non-temporal accesses (default 64 MiB; 0: never). mapped_io_bytes: evaluate() of a graph whose inputs and outputs
 *   are at most this many bytes in all reads and writes them in page-locked host memory instead of copying them
 *   to and from the arena (default 64 KiB; 0: never). stream_weights_bytes: a plan with at least this many bytes of
 *   constants reads the constant right operands of its matmuls (under left operands of up to 1024 rows) with the
 *   non-temporal hint, as streams that cannot stay in the last-level cache from one evaluation to the next (default
 *   256 MiB; 0: never). */
typedef struct {
    size_t struct_bytes; /* sizeof(knhip_executor_options), set by knhip_executor_options_default */
    int plan_only, preserve_inputs, step_by_step;
    int fuse_attention, fuse_gated_matmul, group_matmuls, pack_matmul_constants, pointwise_conv_as_matmul, join_elementwise, split_reduce;
    int tiled_transpose, split_conv_channels, plane_conv_any_width;
    int direct_gemm, split_k, tail_split, dot_products;
    uint64_t streaming_bytes, mapped_io_bytes, stream_weights_bytes;
} knhip_executor_options;
int knhip_executor_options_default(knhip_executor_options *options);

/* CudaExecutor::new(device, &graph, batch_size) (executor.rs:61) */
int knhip_executor_new(int device, const knhip_graph *graph, size_t batch_size, const knhip_executor_options *options,
                       knhip_executor **out);
int knhip_executor_new_from_blob(int device, const uint8_t *blob, size_t len, size_t batch_size,
                                 const knhip_executor_options *options, knhip_executor **out);
void knhip_executor_free(knhip_executor *ex);

int knhip_executor_io_count(const knhip_executor *ex, size_t *inputs, size_t *outputs);
/* dtype, rank and concrete dims (cap entries of room) of input / output `index` */
int knhip_executor_io_info(const knhip_executor *ex, int is_output, size_t index, int *dtype, size_t *rank,
                           size_t *dims, size_t cap);

/* CudaExecutor::evaluate (executor.rs:117-195): dense row-major host buffers in, dense row-major host buffers out.
 * Byte counts are checked against the planned shapes. Every byte is copied once on the host on each side (caller's
 * buffer <-> page-locked staging, straight from and into the caller's buffers); tensors above 2 MiB move in chunks of 2 to 8 MiB, the
 * host copy of one chunk overlapping the bus transfer of another, with the host copies spread over up to four threads
 * (three of them owned by the executor, started by the first evaluation that has 2 MiB or more to copy at once). */
int knhip_executor_evaluate(knhip_executor *ex, const void *const *inputs, const size_t *input_bytes, size_t input_count,
                            void *const *outputs, const size_t *output_bytes, size_t output_count);
/* run_async (executor.rs:199-258): launch all steps on the executor's stream, no synchronisation */
int knhip_executor_run_async(knhip_executor *ex);
/* No counterpart in the reference (its executor launches step by step, executor.rs:199-206): when enabled, run_async
 * and evaluate replay the launch list as one HIP graph, captured on the first run. For graphs of many small kernels,
 * where the launches dominate (tiny MLP at batch 8). Profiled runs still launch step by step. */
int knhip_executor_set_graph_mode(knhip_executor *ex, int enabled);
int knhip_executor_synchronize(knhip_executor *ex);
/* The timing loop of the reference's profile_net (kn-cuda-eval/src/bin/profile_net.rs:146-180, `--skip-io`):
 * `iterations` back-to-back run_async calls bracketed by two HIP events recorded on the executor's stream;
 * returns the elapsed device time in milliseconds for all iterations together. */
int knhip_executor_time_runs(knhip_executor *ex, size_t iterations, float *elapsed_ms);
/* Device addresses of the dense input / output tensors inside the arena (pub device_inputs / device_outputs). Their
 * contents are what run_async reads and writes. evaluate() leaves its inputs and outputs there too, EXCEPT for
 * graphs under the mapped_io_bytes option (64 KiB of inputs + outputs by default), whose evaluate() works on page-locked
 * host memory and never touches these buffers: a caller that mixes evaluate() with device-side reads of these
 * addresses sets mapped_io_bytes to 0. */
int knhip_executor_input_ptr(const knhip_executor *ex, size_t index, void **ptr);
int knhip_executor_output_ptr(const knhip_executor *ex, size_t index, void **ptr);
/* the HIP stream (hipStream_t) every step is launched on (CudaExecutor::stream, executor.rs:112-114) */
int knhip_executor_stream(const knhip_executor *ex, void **stream);

/* set_profile / last_profile (executor.rs:260-266). Seconds per step kind in the order
 * conv, mat_mul, scalar_op, reduce_op, softmax_op, layernorm_op, gather_op. */
typedef struct {
    float per_kind[7];
    float total_cpu, total_gpu, timing_overhead;
    size_t step_count;
} knhip_profile;
int knhip_executor_set_profile(knhip_executor *ex, int enabled);
int knhip_executor_last_profile(const knhip_executor *ex, int *available, knhip_profile *profile);
int knhip_executor_profile_step_seconds(const knhip_executor *ex, float *buf, size_t cap);
int knhip_executor_profile_str(const knhip_executor *ex, char *buf, size_t cap, size_t *needed);

/* MemoryUsage (kn-cuda-eval/src/planner.rs:67-81) */
typedef struct {
    size_t dedicated_bytes, shared_bytes, zero_bytes, hypo_shared_bytes_peak, hypo_shared_bytes_total, arena_bytes;
} knhip_mem_usage;
int knhip_executor_mem_usage(const knhip_executor *ex, knhip_mem_usage *usage);

/* the planned launch list (Debug output of the executor, executor.rs:269-289) */
int knhip_executor_step_count(const knhip_executor *ex, size_t *count);
/* kind: 0 conv, 1 mat_mul, 2 scalar_op, 3 reduce_op, 4 softmax_op, 5 layernorm_op, 6 gather_op */
int knhip_executor_step_kind(const knhip_executor *ex, size_t index, int *kind);
int knhip_executor_step_str(const knhip_executor *ex, size_t index, char *buf, size_t cap, size_t *needed);
/* algorithmic work of one launch of the step, for roofline reports next to the per-step times of the profile
 * (the role of the per-kernel lines of kn-cuda-eval/src/executor.rs:269-289 and profile_net.rs:147-171):
 * flops = 2 * multiply-adds of a conv / mat_mul step (0 for the others), bytes = every distinct operand element once */
int knhip_executor_step_work(const knhip_executor *ex, size_t index, double *flops, double *bytes);
int knhip_executor_step_source(const knhip_executor *ex, size_t index, char *buf, size_t cap, size_t *needed);
/* No counterpart in the reference. A plan of a few tiny steps (each small enough for a single workgroup) is also
 * compiled into ONE kernel that runs the steps in launch order; run_async and evaluate launch it instead of the steps
 * unless the run is profiled. The source of that kernel, or an empty string when the plan is launched step by step. */
int knhip_executor_fused_source(const knhip_executor *ex, char *buf, size_t cap, size_t *needed);
int knhip_executor_str(const knhip_executor *ex, char *buf, size_t cap, size_t *needed);

/* Layout algebra hooks for tests (kn-cuda-eval/src/shape.rs:25-285). Strides are in elements.
 * flags: *simple = row-major contiguous, *dense = covers its span exactly once in some axis order (shape.rs:67-73).
 * view: *ok = 0 when the view cannot be expressed as a stride edit (shape.rs:135-189).
 * slice: shape.rs:83-96. Output arrays need `rank` (view: `new_rank`) entries. */
int knhip_strided_flags(const size_t *shape, const int64_t *strides, size_t rank, int *simple, int *dense);
int knhip_strided_view(const size_t *shape, const int64_t *strides, size_t rank, const size_t *new_shape,
                       size_t new_rank, int *ok, int64_t *new_strides);
int knhip_strided_slice(const size_t *shape, const int64_t *strides, size_t rank, size_t axis, size_t start, size_t end,
                        size_t step, size_t *out_shape, int64_t *out_strides);

/* kernel compile cache counters (autokernel/common.rs:14-46) */
int knhip_compile_stats(size_t *compiled, size_t *memory_hits, size_t *disk_hits);

#ifdef __cplusplus
}
#endif

#endif /* KNHIP_H */
