//! The flat little-endian form in which a `kn_graph::graph::Graph` crosses the C ABI
//! (`knhip_executor_new_from_blob`). Produced by walking the public graph API only
//! (`Graph::values`, `graph[value]`, `inputs`, `outputs`: kn-graph/src/graph.rs:354-394).
//!
//! ```text
//! u32 magic "KNHG", u32 version = 1
//! u32 value_count, then per value:
//!   u8 dtype, u32 rank, rank x (u64 fixed_factor, u32 batch_exp), u8 operation, payload, u32 debug_id_len, bytes
//! u32 input_count, values; u32 output_count, values
//! ```
use kn_graph::dispatch_dtensor;
use kn_graph::dtype::{DTensor, DType};
use kn_graph::graph::{BinaryOp, Graph, Operation, ReduceOp, UnaryOp, Value};

pub const MAGIC: &[u8; 4] = b"KNHG";
pub const VERSION: u32 = 1;

/// The element type codes of knhip.h (`KNHIP_F32` ... `KNHIP_BOOL`), in the order of dtype.rs:24-37.
pub fn dtype_code(dtype: DType) -> u8 {
    match dtype {
        DType::F32 => 0,
        DType::F64 => 1,
        DType::I8 => 2,
        DType::I16 => 3,
        DType::I32 => 4,
        DType::I64 => 5,
        DType::U8 => 6,
        DType::U16 => 7,
        DType::U32 => 8,
        DType::U64 => 9,
        DType::Bool => 10,
    }
}

pub fn dtype_from_code(code: i32) -> DType {
    match code {
        0 => DType::F32,
        1 => DType::F64,
        2 => DType::I8,
        3 => DType::I16,
        4 => DType::I32,
        5 => DType::I64,
        6 => DType::U8,
        7 => DType::U16,
        8 => DType::U32,
        9 => DType::U64,
        10 => DType::Bool,
        _ => panic!("element type code {} has no kn-graph DType (F16 needs a DType::F16 variant first)", code),
    }
}

/// (operation code, cast target; 0 for operations that are no cast): graph.rs:173-195 in declaration order, then the two casts.
pub fn unary_code(op: UnaryOp) -> (u8, u8) {
    match op {
        UnaryOp::Abs => (0, 0),
        UnaryOp::Neg => (1, 0),
        UnaryOp::Sin => (2, 0),
        UnaryOp::Cos => (3, 0),
        UnaryOp::Exp => (4, 0),
        UnaryOp::Log => (5, 0),
        UnaryOp::Sqrt => (6, 0),
        UnaryOp::Sigmoid => (7, 0),
        UnaryOp::Tanh => (8, 0),
        UnaryOp::Erf => (9, 0),
        UnaryOp::Mish => (10, 0),
        UnaryOp::Softplus => (11, 0),
        UnaryOp::ValueCast(to) => (12, dtype_code(to)),
        UnaryOp::BitCast(to) => (13, dtype_code(to)),
    }
}

pub fn binary_code(op: BinaryOp) -> u8 {
    match op {
        BinaryOp::Add => 0,
        BinaryOp::Sub => 1,
        BinaryOp::Mul => 2,
        BinaryOp::Div => 3,
        BinaryOp::Min => 4,
        BinaryOp::Max => 5,
        BinaryOp::Pow => 6,
    }
}

pub fn reduce_code(op: ReduceOp) -> u8 {
    match op {
        ReduceOp::Sum => 0,
        ReduceOp::Mean => 1,
        ReduceOp::Prod => 2,
        ReduceOp::Max => 3,
        ReduceOp::Min => 4,
    }
}

/// The elements of a tensor in row-major order as little-endian bytes (bools as one byte, 0 or 1).
pub fn dense_le_bytes(tensor: &DTensor) -> Vec<u8> {
    match tensor {
        DTensor::Bool(tensor) => tensor.iter().map(|b| b.0 as u8).collect(),
        _ => dispatch_dtensor!(tensor, |T, _f, inner| {
            let dense = inner.as_standard_layout();
            let slice: &[T] = dense.as_slice().expect("standard layout is contiguous");
            // the targets of both sides are little endian; to_le_bytes per element would spell the same bytes
            unsafe { std::slice::from_raw_parts(slice.as_ptr() as *const u8, std::mem::size_of_val(slice)) }.to_vec()
        }),
    }
}

struct Writer {
    out: Vec<u8>,
}

impl Writer {
    fn u8(&mut self, v: u8) {
        self.out.push(v);
    }
    fn u32(&mut self, v: usize) {
        let v = u32::try_from(v).expect("value does not fit the 32 bit field of the graph blob");
        self.out.extend_from_slice(&v.to_le_bytes());
    }
    fn u64(&mut self, v: usize) {
        self.out.extend_from_slice(&(v as u64).to_le_bytes());
    }
    fn value(&mut self, v: Value) {
        self.u32(v.index());
    }
}

pub fn serialize_graph(graph: &Graph) -> Vec<u8> {
    let mut w = Writer { out: Vec::new() };
    w.out.extend_from_slice(MAGIC);
    w.u32(VERSION as usize);

    let values: Vec<Value> = graph.values().collect();
    w.u32(values.len());
    for (position, &value) in values.iter().enumerate() {
        // values are numbered densely in creation order (graph.rs:86-91): operands always precede their users
        assert_eq!(value.index(), position);
        let info = &graph[value];

        w.u8(dtype_code(info.dtype));
        w.u32(info.shape.rank());
        for size in &info.shape.dims {
            let (fixed_factor, batch_exp) = size.components_factor_exp();
            w.u64(fixed_factor);
            w.u32(batch_exp as usize);
        }

        match &info.operation {
            &Operation::Input { index } => {
                w.u8(0);
                w.u32(index);
            }
            Operation::Constant { tensor } => {
                w.u8(1);
                let bytes = dense_le_bytes(tensor);
                w.u64(bytes.len());
                w.out.extend_from_slice(&bytes);
            }
            &Operation::View { input } => {
                w.u8(2);
                w.value(input);
            }
            &Operation::Broadcast { input } => {
                w.u8(3);
                w.value(input);
            }
            Operation::Permute { input, permutation } => {
                w.u8(4);
                w.value(*input);
                w.u32(permutation.len());
                for &axis in permutation {
                    w.u32(axis);
                }
            }
            &Operation::Slice { input, axis, range } => {
                w.u8(5);
                w.value(input);
                w.u32(axis);
                w.u64(range.start);
                w.u64(range.end);
                w.u64(range.step);
            }
            &Operation::Flip { input, axis } => {
                w.u8(6);
                w.value(input);
                w.u32(axis);
            }
            &Operation::Gather { input, axis, indices } => {
                w.u8(7);
                w.value(input);
                w.u32(axis);
                w.value(indices);
            }
            Operation::Concat { inputs, axis } => {
                w.u8(8);
                w.u32(inputs.len());
                for &input in inputs {
                    w.value(input);
                }
                w.u32(*axis);
            }
            &Operation::Conv { input, filter, details } => {
                w.u8(9);
                w.value(input);
                w.value(filter);
                for x in [
                    details.stride_y,
                    details.stride_x,
                    details.padding_y,
                    details.padding_x,
                    details.kernel_h,
                    details.kernel_w,
                    details.output_h,
                    details.output_w,
                ] {
                    w.u64(x);
                }
            }
            &Operation::MatMul { left, right } => {
                w.u8(10);
                w.value(left);
                w.value(right);
            }
            &Operation::Unary { input, op } => {
                w.u8(11);
                w.value(input);
                let (code, cast) = unary_code(op);
                w.u8(code);
                w.u8(cast);
            }
            &Operation::Binary { left, right, op } => {
                w.u8(12);
                w.value(left);
                w.value(right);
                w.u8(binary_code(op));
            }
            &Operation::Softmax { input, axis } => {
                w.u8(13);
                w.value(input);
                w.u32(axis);
            }
            &Operation::Layernorm { input, axis, eps } => {
                w.u8(14);
                w.value(input);
                w.u32(axis);
                w.out.extend_from_slice(&eps.into_inner().to_le_bytes());
            }
            Operation::Reduce { input, axes, op } => {
                w.u8(15);
                w.value(*input);
                w.u32(axes.len());
                for &axis in axes {
                    w.u32(axis);
                }
                w.u8(reduce_code(*op));
            }
        }

        w.u32(info.debug_id.len());
        w.out.extend_from_slice(info.debug_id.as_bytes());
    }

    w.u32(graph.inputs().len());
    for &input in graph.inputs() {
        w.value(input);
    }
    w.u32(graph.outputs().len());
    for &output in graph.outputs() {
        w.value(output);
    }
    w.out
}
