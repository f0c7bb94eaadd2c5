//! `StridedShape`: a shape with element strides (zero = broadcast, negative = flipped), the twin of
//! kn-cuda-eval/src/shape.rs:25-285. The two operations with real logic in them, `view` and `slice`, and the
//! simple / dense tests are computed by the library (`knhip_strided_*`), which keeps the rules in one place.
use std::os::raw::c_int;

use kn_graph::graph::SliceRange;
use kn_hip_sys::wrapper::Status;
use kn_hip_sys::{knhip_strided_flags, knhip_strided_slice, knhip_strided_view};

#[derive(Debug, Clone, Eq, PartialEq, Hash)]
pub struct StridedShape {
    shape: Vec<usize>,
    strides: Vec<isize>,
    has_simple_strides: bool,
    has_dense_strides: bool,
}

#[derive(Debug, Clone, Eq, PartialEq)]
pub struct ViewError {
    pub old: StridedShape,
    pub new: Vec<usize>,
}

impl StridedShape {
    pub fn new(shape: Vec<usize>, strides: Vec<isize>) -> Self {
        assert_eq!(shape.len(), strides.len(), "Shape and stride rank mismatch");
        let strides64: Vec<i64> = strides.iter().map(|&s| s as i64).collect();
        let (mut simple, mut dense): (c_int, c_int) = (0, 0);
        unsafe { knhip_strided_flags(shape.as_ptr(), strides64.as_ptr(), shape.len(), &mut simple, &mut dense) }.unwrap();
        StridedShape { shape, strides, has_simple_strides: simple != 0, has_dense_strides: dense != 0 }
    }

    pub fn new_simple(shape: Vec<usize>) -> Self {
        let mut strides = vec![0isize; shape.len()];
        let mut run = 1isize;
        for (stride, &dim) in strides.iter_mut().zip(&shape).rev() {
            *stride = run;
            run *= dim as isize;
        }
        StridedShape::new(shape, strides)
    }

    pub fn shape(&self) -> &[usize] {
        &self.shape
    }

    pub fn strides(&self) -> &[isize] {
        &self.strides
    }

    pub fn rank(&self) -> usize {
        self.shape.len()
    }

    pub fn size(&self) -> usize {
        self.shape.iter().product()
    }

    pub fn has_simple_strides(&self) -> bool {
        self.has_simple_strides
    }

    pub fn has_dense_strides(&self) -> bool {
        self.has_dense_strides
    }

    pub(crate) fn strides_i64(&self) -> Vec<i64> {
        self.strides.iter().map(|&s| s as i64).collect()
    }

    pub fn permute(&self, permutation: &[usize]) -> StridedShape {
        assert_eq!(permutation.len(), self.rank(), "Permutation rank mismatch");
        let mut seen = vec![false; self.rank()];
        for &p in permutation {
            assert!(p < self.rank() && !seen[p], "Invalid permutation {:?}", permutation);
            seen[p] = true;
        }
        StridedShape::new(permutation.iter().map(|&p| self.shape[p]).collect(), permutation.iter().map(|&p| self.strides[p]).collect())
    }

    pub fn view(&self, new_shape: Vec<usize>) -> Result<StridedShape, ViewError> {
        let mut ok: c_int = 0;
        let mut new_strides = vec![0i64; new_shape.len().max(1)];
        unsafe {
            knhip_strided_view(
                self.shape.as_ptr(),
                self.strides_i64().as_ptr(),
                self.rank(),
                new_shape.as_ptr(),
                new_shape.len(),
                &mut ok,
                new_strides.as_mut_ptr(),
            )
        }
        .unwrap();
        if ok == 0 {
            return Err(ViewError { old: self.clone(), new: new_shape });
        }
        let strides = new_strides[..new_shape.len()].iter().map(|&s| s as isize).collect();
        Ok(StridedShape::new(new_shape, strides))
    }

    pub fn broadcast(&self, new_shape: Vec<usize>) -> StridedShape {
        assert!(new_shape.len() >= self.rank(), "Cannot broadcast {:?} to {:?}", self, new_shape);
        let pad = new_shape.len() - self.rank();
        let mut strides = vec![0isize; pad];
        for (i, &new_dim) in new_shape[pad..].iter().enumerate() {
            if self.shape[i] == new_dim {
                strides.push(self.strides[i]);
            } else {
                assert_eq!(self.shape[i], 1, "Cannot broadcast {:?} to {:?}", self, new_shape);
                strides.push(0);
            }
        }
        StridedShape::new(new_shape, strides)
    }

    pub fn slice(&self, axis: usize, range: SliceRange) -> StridedShape {
        assert!(axis < self.rank(), "Slice axis {} out of bounds for {:?}", axis, self);
        let mut out_shape = vec![0usize; self.rank()];
        let mut out_strides = vec![0i64; self.rank()];
        unsafe {
            knhip_strided_slice(
                self.shape.as_ptr(),
                self.strides_i64().as_ptr(),
                self.rank(),
                axis,
                range.start,
                range.end,
                range.step,
                out_shape.as_mut_ptr(),
                out_strides.as_mut_ptr(),
            )
        }
        .unwrap();
        StridedShape::new(out_shape, out_strides.iter().map(|&s| s as isize).collect())
    }

    pub fn flip(&self, axis: usize) -> StridedShape {
        let mut strides = self.strides.clone();
        strides[axis] = -strides[axis];
        StridedShape::new(self.shape.clone(), strides)
    }

    pub fn repeat_unary(&self, axis: usize, count: usize) -> StridedShape {
        assert_eq!(self.shape[axis], 1, "repeat_unary needs a unit axis");
        let (mut shape, mut strides) = (self.shape.clone(), self.strides.clone());
        shape[axis] = count;
        strides[axis] = 0;
        StridedShape::new(shape, strides)
    }

    pub fn remove(&self, axis: usize) -> StridedShape {
        let (mut shape, mut strides) = (self.shape.clone(), self.strides.clone());
        shape.remove(axis);
        strides.remove(axis);
        StridedShape::new(shape, strides)
    }
}
