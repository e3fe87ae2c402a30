//! sliced's op traits for `HIP<Mods>`, f32 only: every method is one call into the C ABI.  Each impl
//! names the trait's file in the reference; the bodies follow the reference's OpenCL device
//! (`retrieve` the output, launch, return), e.g. src/ops2/gemm/opencl.rs:13-27.
//!
//! Set or accumulate: the gradient traits accumulate (`+=`) as the reference's CPU bodies do, except
//! gemm_grad, softmax_grad and transpose_grad, which overwrite there (BLAS beta = 0,
//! src/ops2/gemm/grad/cpu_stack.rs:36-39; src/ops2/transpose/cpu.rs:22-23) and take GRAD_BETA here.
use custos::{
    AddOperation, ApplyFunction, Buffer, Device, Eval, MayToCLSource, OnDropBuffer, Resolve, Retrieve, Retriever, Shape,
    UnaryGrad,
};
use sliced::{
    assign_or_set::{AssignOrSet, Set},
    AddElementWiseGrad, BinaryElementWise, BinaryElementWiseGrad, ColOp, ColOpGrad, Diagflat, DiagflatGrad, Gemm, GemmGrad,
    Max, MaxCols, MaxColsGrad, MaxRows, MaxRowsGrad, Mean, MeanCols, MeanColsGrad, MeanRows, MeanRowsGrad, Onehot, RowOp,
    RowOpGrad, Softmax, SoftmaxGrad, Sum, SumCols, SumColsGrad, SumRows, SumRowsGrad, TranposeGrad, Transpose,
};

use crate::{check, ffi::*, probe, HIP};

/// 0 = overwrite (the reference's CPU device), 1 = accumulate (its OpenCL device,
/// src/ops2/gemm/grad/opencl.rs:20,33).
pub const GRAD_BETA: f32 = 0.0;

type Buf<'a, Mods, S = ()> = Buffer<'a, f32, HIP<Mods>, S>;

// ------------------------------------------------------------------------------------ gemm
// src/ops2/gemm/mod.rs:21-32
impl<Mods: Retrieve<Self, f32> + 'static> Gemm<f32> for HIP<Mods> {
    #[inline]
    fn gemm(&self, m: usize, k: usize, n: usize, lhs: &Buf<Mods>, rhs: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(m * n, (lhs, rhs)).unwrap();
        check(unsafe { slhip_gemm(self.ctx, m, k, n, lhs.ptr(), rhs.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}

// src/ops2/gemm/grad.rs:15-29.  A null pointer stands for `!requires_grad()`
// (src/ops2/gemm/grad/cpu_stack.rs:35,38).
impl<Mods: OnDropBuffer + 'static> GemmGrad<f32> for HIP<Mods> {
    fn gemm_grad(
        &self,
        m: usize,
        k: usize,
        n: usize,
        lhs: &Buf<Mods>,
        rhs: &Buf<Mods>,
        lhs_grad: &mut Buf<Mods>,
        rhs_grad: &mut Buf<Mods>,
        out_grad: &Buf<Mods>,
    ) {
        let lg = if lhs.requires_grad() { lhs_grad.ptr_mut() } else { core::ptr::null_mut() };
        let rg = if rhs.requires_grad() { rhs_grad.ptr_mut() } else { core::ptr::null_mut() };
        check(unsafe { slhip_gemm_grad(self.ctx, m, k, n, lhs.ptr(), rhs.ptr(), lg, rg, out_grad.ptr(), GRAD_BETA) }).unwrap();
    }
}

// ------------------------------------------------------------------------------------ reductions
// src/ops2/sum/mod.rs:15-25.  *_rows reduces OVER the rows (output length = cols), *_cols over the
// columns (output length = rows): the reference's naming.
impl<Mods: OnDropBuffer + 'static> Sum<f32> for HIP<Mods> {
    fn sum(&self, x: &Buf<Mods>) -> f32 {
        self.scalar(x, slhip_sum)
    }
}
impl<Mods: OnDropBuffer + 'static> Max<f32> for HIP<Mods> {
    fn max(&self, x: &Buf<Mods>) -> f32 {
        self.scalar(x, slhip_max)
    }
}
impl<Mods: OnDropBuffer + 'static, S: Shape> Mean<f32, S> for HIP<Mods> {
    fn mean(&self, x: &Buf<Mods, S>) -> f32 {
        let mut host = 0.0f32;
        let mut dev: *mut core::ffi::c_void = core::ptr::null_mut();
        unsafe {
            check(slhip_malloc(self.ctx, 4, &mut dev)).unwrap();
            check(slhip_mean(self.ctx, x.len(), x.ptr(), dev as *mut f32)).unwrap();
            check(slhip_memcpy_d2h(self.ctx, &mut host as *mut f32 as *mut _, dev, 4)).unwrap();
            slhip_free(self.ctx, dev);
        }
        host
    }
}
impl<Mods> HIP<Mods> {
    fn scalar<S: Shape>(
        &self,
        x: &Buffer<f32, Self, S>,
        f: unsafe extern "C" fn(*mut SlhipCtx, usize, *const f32, *mut f32) -> i32,
    ) -> f32
    where
        Self: Device,
    {
        let mut host = 0.0f32;
        let mut dev: *mut core::ffi::c_void = core::ptr::null_mut();
        unsafe {
            check(slhip_malloc(self.ctx, 4, &mut dev)).unwrap();
            check(f(self.ctx, x.len(), x.ptr(), dev as *mut f32)).unwrap();
            check(slhip_memcpy_d2h(self.ctx, &mut host as *mut f32 as *mut _, dev, 4)).unwrap();
            slhip_free(self.ctx, dev);
        }
        host
    }
}

macro_rules! reduction {
    ($trait:ident, $method:ident, $ffi:ident, over_rows = $over_rows:expr) => {
        impl<Mods: Retrieve<Self, f32> + 'static> $trait<f32> for HIP<Mods> {
            #[inline]
            fn $method(&self, cols: usize, x: &Buf<Mods>) -> Buf<Mods> {
                let rows = x.len() / cols;
                let mut out = self.retrieve(if $over_rows { cols } else { rows }, x).unwrap();
                check(unsafe { $ffi(self.ctx, rows, cols, x.ptr(), out.ptr_mut()) }).unwrap();
                out
            }
        }
    };
}
reduction!(SumRows, sum_rows, slhip_sum_rows, over_rows = true); // src/ops2/sum/mod.rs:19-21
reduction!(SumCols, sum_cols, slhip_sum_cols, over_rows = false); // :23-25
reduction!(MaxRows, max_rows, slhip_max_rows, over_rows = true); // src/ops2/max/mod.rs:20-22
reduction!(MeanRows, mean_rows, slhip_mean_rows, over_rows = true); // src/ops2/mean/mod.rs:19-31
reduction!(MeanCols, mean_cols, slhip_mean_cols, over_rows = false); // :33-45

// src/ops2/max/mod.rs:24-26 (takes rows as well)
impl<Mods: Retrieve<Self, f32> + 'static> MaxCols<f32> for HIP<Mods> {
    #[inline]
    fn max_cols(&self, rows: usize, cols: usize, x: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(rows, x).unwrap();
        check(unsafe { slhip_max_cols(self.ctx, rows, cols, x.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}

macro_rules! broadcast_grad {
    ($trait:ident, $method:ident, $ffi:ident) => {
        impl<Mods: OnDropBuffer + 'static> $trait<f32> for HIP<Mods> {
            #[inline]
            fn $method(&self, cols: usize, x_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
                let rows = x_grad.len() / cols;
                check(unsafe { $ffi(self.ctx, rows, cols, x_grad.ptr_mut(), out_grad.ptr()) }).unwrap();
            }
        }
    };
}
broadcast_grad!(SumRowsGrad, sum_rows_grad, slhip_sum_rows_grad); // src/ops2/sum/grad.rs:7-14
broadcast_grad!(SumColsGrad, sum_cols_grad, slhip_sum_cols_grad); // :16-23
broadcast_grad!(MeanRowsGrad, mean_rows_grad, slhip_mean_rows_grad); // src/ops2/mean/grad.rs
broadcast_grad!(MeanColsGrad, mean_cols_grad, slhip_mean_cols_grad);

macro_rules! max_grad {
    ($trait:ident, $method:ident, $ffi:ident) => {
        // src/ops2/max/grad.rs: max_rows_grad reaches every tied row, max_cols_grad only the first
        // tied column (src/ops2/max/grad/cpu.rs:40-69)
        impl<Mods: OnDropBuffer + 'static> $trait<f32> for HIP<Mods> {
            #[inline]
            fn $method(&self, cols: usize, out: &Buf<Mods>, x: &Buf<Mods>, x_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
                let rows = x.len() / cols;
                check(unsafe { $ffi(self.ctx, rows, cols, out.ptr(), x.ptr(), x_grad.ptr_mut(), out_grad.ptr()) }).unwrap();
            }
        }
    };
}
max_grad!(MaxRowsGrad, max_rows_grad, slhip_max_rows_grad);
max_grad!(MaxColsGrad, max_cols_grad, slhip_max_cols_grad);

// ------------------------------------------------------------------------------------ softmax
// src/ops2/softmax/mod.rs:16-18: one pass instead of the CPU body's five (src/ops2/softmax/cpu.rs:11-16)
impl<Mods: Retrieve<Self, f32> + 'static> Softmax<f32> for HIP<Mods> {
    #[inline]
    fn softmax(&self, samples: usize, features: usize, x: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(x.len(), x).unwrap();
        check(unsafe { slhip_softmax(self.ctx, samples, features, x.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}
// src/ops2/softmax/grad.rs:15-24: the closed form s * (g - <s, g>) of the CPU body's per-sample Jacobian
impl<Mods: OnDropBuffer + 'static> SoftmaxGrad<f32> for HIP<Mods> {
    #[inline]
    fn softmax_grad(&self, samples: usize, features: usize, x_grad: &mut Buf<Mods>, out: &Buf<Mods>, out_grad: &Buf<Mods>) {
        check(unsafe {
            slhip_softmax_grad(self.ctx, samples, features, x_grad.ptr_mut(), out.ptr(), out_grad.ptr(), GRAD_BETA)
        })
        .unwrap();
    }
}

// ------------------------------------------------------------------------------------ transpose
// src/ops2/transpose/mod.rs:17-21; AOS = Set overwrites, Assign adds (src/assign_or_set.rs)
impl<Mods: Retrieve<Self, f32> + 'static, AOS: AssignOrSet<f32>> Transpose<f32, (), (), Self, AOS> for HIP<Mods> {
    #[inline]
    fn transpose(&self, rows: usize, cols: usize, x: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(x.len(), x).unwrap();
        check(unsafe { slhip_transpose(self.ctx, rows, cols, x.ptr(), out.ptr_mut(), 0.0) }).unwrap();
        out
    }
}
// src/ops2/transpose/grad.rs:13-26: x_grad[rows x cols] <- transpose of out_grad[cols x rows]
impl<Mods: OnDropBuffer + 'static> TranposeGrad<f32> for HIP<Mods> {
    #[inline]
    fn transpose_grad(&self, rows: usize, cols: usize, x_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
        check(unsafe { slhip_transpose(self.ctx, cols, rows, out_grad.ptr(), x_grad.ptr_mut(), GRAD_BETA) }).unwrap();
    }
}

// ------------------------------------------------------------------------------------ row op
// src/ops2/row_op/mod.rs:17-47.  The closure form is `|out, lhs, rhs| *out = lhs op rhs`: probed.
impl<Mods: Retrieve<Self, f32> + 'static> RowOp<f32> for HIP<Mods> {
    fn row_op<F: Fn(&mut f32, f32, f32) + Copy>(&self, cols: usize, lhs: &Buf<Mods>, rhs: &Buf<Mods>, f: F) -> Buf<Mods> {
        let as_fn = |a: f32, b: f32| {
            let mut c = 0.0;
            f(&mut c, a, b);
            c
        };
        let op = [(SLHIP_ADD, 8.0f32), (SLHIP_SUB, -2.0), (SLHIP_MUL, 15.0), (SLHIP_DIV, 0.6)]
            .iter()
            .find(|(_, want)| (as_fn(3.0, 5.0) - want).abs() < 1e-6)
            .map(|(op, _)| *op)
            .expect("row_op: only add, sub, mul and div closures have a device kernel");
        let mut out = self.retrieve(lhs.len(), (lhs, rhs)).unwrap();
        check(unsafe { slhip_row_op(self.ctx, op, lhs.len() / cols, cols, lhs.ptr(), rhs.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
    #[inline]
    fn add_row(&self, cols: usize, lhs: &Buf<Mods>, rhs: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(lhs.len(), (lhs, rhs)).unwrap();
        check(unsafe { slhip_add_row(self.ctx, lhs.len() / cols, cols, lhs.ptr(), rhs.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
    #[inline]
    fn add_row_mut(&self, rows: usize, cols: usize, lhs: &mut Buf<Mods>, rhs: &Buf<Mods>) {
        // out == lhs is the documented in-place form
        check(unsafe { slhip_add_row(self.ctx, rows, cols, lhs.ptr(), rhs.ptr(), lhs.ptr_mut()) }).unwrap();
    }
}
// src/ops2/row_op/grad.rs:12-41
impl<Mods: OnDropBuffer + 'static> RowOpGrad<f32> for HIP<Mods> {
    fn row_op_grad(
        &self,
        cols: usize,
        lhs: &Buf<Mods>,
        rhs: &Buf<Mods>,
        lhs_grad: &mut Buf<Mods>,
        rhs_grad: &mut Buf<Mods>,
        out_grad: &Buf<Mods>,
        lhs_grad_fn: impl Fn(f32) -> f32,
        rhs_grad_fn: impl Fn(f32) -> f32,
    ) {
        // the closures are d/dlhs as a function of rhs and d/drhs as a function of lhs
        // (src/ops2/row_op/grad/cpu.rs:66-88): add gives (1, 1), mul gives (rhs, lhs)
        let op = if lhs_grad_fn(3.0) == 1.0 && rhs_grad_fn(5.0) == 1.0 {
            SLHIP_ADD
        } else if lhs_grad_fn(3.0) == 1.0 && rhs_grad_fn(5.0) == -1.0 {
            SLHIP_SUB
        } else if lhs_grad_fn(3.0) == 3.0 && rhs_grad_fn(5.0) == 5.0 {
            SLHIP_MUL
        } else {
            panic!("row_op_grad: only the gradients of add, sub and mul have a device kernel")
        };
        check(unsafe {
            slhip_row_op_grad(self.ctx, op, lhs.len() / cols, cols, lhs.ptr(), rhs.ptr(), lhs_grad.ptr_mut(), rhs_grad.ptr_mut(), out_grad.ptr())
        })
        .unwrap();
    }
    #[inline]
    fn add_row_grad(&self, rows: usize, cols: usize, lhs_grad: &mut Buf<Mods>, rhs_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
        check(unsafe { slhip_add_row_grad(self.ctx, rows, cols, lhs_grad.ptr_mut(), rhs_grad.ptr_mut(), out_grad.ptr()) }).unwrap();
    }
    #[inline]
    fn add_row_mut_grad(&self, rows: usize, cols: usize, rhs_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
        check(unsafe { slhip_add_row_mut_grad(self.ctx, rows, cols, rhs_grad.ptr_mut(), out_grad.ptr()) }).unwrap();
    }
}

// ------------------------------------------------------------------------------------ col op
// src/ops2/col_op/mod.rs:20-57 (sub_cols, div_cols are its provided methods)
impl<Mods: Retrieve<Self, f32> + 'static> ColOp<f32> for HIP<Mods> {
    fn col_op<F>(&self, cols: usize, lhs: &Buf<Mods>, rhs: &Buf<Mods>, f: F) -> Buf<Mods>
    where
        F: Fn(f32, f32) -> f32 + Copy + 'static,
    {
        let op = [(SLHIP_ADD, 8.0f32), (SLHIP_SUB, -2.0), (SLHIP_MUL, 15.0), (SLHIP_DIV, 0.6)]
            .iter()
            .find(|(_, want)| (f(3.0, 5.0) - want).abs() < 1e-6)
            .map(|(op, _)| *op)
            .expect("col_op: only add, sub, mul and div closures have a device kernel");
        let mut out = self.retrieve(lhs.len(), (lhs, rhs)).unwrap();
        check(unsafe { slhip_col_op(self.ctx, op, lhs.len() / cols, cols, lhs.ptr(), rhs.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}
// src/ops2/col_op/grad.rs:12-27 (the method is called row_op_grad there as well)
impl<Mods: OnDropBuffer + 'static> ColOpGrad<f32> for HIP<Mods> {
    fn row_op_grad<LhsGrad, RhsGrad>(
        &self,
        cols: usize,
        lhs: &Buf<Mods>,
        rhs: &Buf<Mods>,
        lhs_grad: &mut Buf<Mods>,
        rhs_grad: &mut Buf<Mods>,
        out_grad: &Buf<Mods>,
        lhs_grad_fn: impl Fn(Resolve<f32>, Resolve<f32>) -> LhsGrad,
        rhs_grad_fn: impl Fn(Resolve<f32>, Resolve<f32>) -> RhsGrad,
    ) where
        LhsGrad: Eval<f32> + ToString,
        RhsGrad: Eval<f32> + ToString,
    {
        let op = probe::binary_op_of_grads(lhs_grad_fn, rhs_grad_fn)
            .expect("col_op gradient: only add, sub, mul and div have a device kernel");
        check(unsafe {
            slhip_col_op_grad(self.ctx, op, lhs.len() / cols, cols, lhs.ptr(), rhs.ptr(), lhs_grad.ptr_mut(), rhs_grad.ptr_mut(), out_grad.ptr())
        })
        .unwrap();
    }
}

// ------------------------------------------------------------------------------------ elementwise
// src/ops2/binary_ew/mod.rs:55-100
impl<Mods: Retrieve<Self, f32, S> + 'static, S: Shape> BinaryElementWise<f32, S> for HIP<Mods> {
    fn binary_ew<O>(&self, lhs: &Buf<Mods, S>, rhs: &Buf<Mods, S>, f: impl Fn(Resolve<f32>, Resolve<f32>) -> O + Copy + 'static) -> Buf<Mods, S>
    where
        O: Eval<f32> + MayToCLSource,
    {
        let op = probe::binary_op(f).expect("binary_ew: only add, sub, mul and div have a device kernel");
        let mut out = self.retrieve(lhs.len(), (lhs, rhs)).unwrap();
        check(unsafe { slhip_ew_binary(self.ctx, op, lhs.len(), lhs.ptr(), rhs.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}
// src/ops2/binary_ew/grad.rs:23-36
impl<Mods: OnDropBuffer + 'static, S: Shape> BinaryElementWiseGrad<f32, S> for HIP<Mods> {
    fn binary_ew_grad<LO, RO>(
        &self,
        lhs: &Buf<Mods, S>,
        rhs: &Buf<Mods, S>,
        lhs_grad: &mut Buf<Mods, S>,
        rhs_grad: &mut Buf<Mods, S>,
        out: &Buf<Mods, S>,
        lhs_grad_fn: impl Fn(Resolve<f32>, Resolve<f32>) -> LO,
        rhs_grad_fn: impl Fn(Resolve<f32>, Resolve<f32>) -> RO,
    ) where
        LO: Eval<f32> + MayToCLSource,
        RO: Eval<f32> + MayToCLSource,
    {
        let op = probe::binary_op_of_grads(lhs_grad_fn, rhs_grad_fn)
            .expect("binary_ew_grad: only the gradients of add, sub, mul and div have a device kernel");
        let (lg, rg) = (lhs_grad.ptr_mut(), rhs_grad.ptr_mut());
        if lg == rg {
            // x op x: lhs term first, then the rhs term, into the one gradient
            // (slice_binary_grad, src/ops2/binary_ew/grad/cpu_stack.rs:55-58)
            check(unsafe { slhip_ew_binary_grad(self.ctx, op, lhs.len(), lhs.ptr(), rhs.ptr(), lg, core::ptr::null_mut(), out.ptr()) }).unwrap();
            check(unsafe { slhip_ew_binary_grad(self.ctx, op, lhs.len(), lhs.ptr(), rhs.ptr(), core::ptr::null_mut(), rg, out.ptr()) }).unwrap();
        } else {
            check(unsafe { slhip_ew_binary_grad(self.ctx, op, lhs.len(), lhs.ptr(), rhs.ptr(), lg, rg, out.ptr()) }).unwrap();
        }
    }
}
// src/ops2/binary_ew/grad.rs:38-46: both gradients += out_grad
impl<Mods: OnDropBuffer + 'static, S: Shape> AddElementWiseGrad<f32, S> for HIP<Mods> {
    fn add_ew_grad(&self, lhs_grad: &mut Buf<Mods, S>, rhs_grad: &mut Buf<Mods, S>, out: &Buf<Mods, S>) {
        let n = out.len();
        // the operand values do not enter add's gradient: out stands in for both
        check(unsafe { slhip_ew_binary_grad(self.ctx, SLHIP_ADD, n, out.ptr(), out.ptr(), lhs_grad.ptr_mut(), rhs_grad.ptr_mut(), out.ptr()) })
            .unwrap();
    }
}

// custos: ApplyFunction::apply_fn / UnaryGrad::add_unary_grad are what square, pow, relu, exp, clip,
// tanh and sigmoid go through (src/ops.rs:36-41,65-72,395,423,438; src/matrix.rs:181-187,218-223,246-255)
impl<Mods: Retrieve<Self, f32, S> + AddOperation + 'static, S: Shape> ApplyFunction<f32, S> for HIP<Mods> {
    fn apply_fn<F>(&self, buf: &Buf<Mods, S>, f: impl Fn(Resolve<f32>) -> F + Copy + 'static) -> Buf<Mods, S>
    where
        F: Eval<f32> + MayToCLSource,
    {
        let (op, p, q) = probe::unary_op(f).expect("apply_fn: this expression has no device kernel");
        let mut out = self.retrieve(buf.len(), buf).unwrap();
        check(unsafe { slhip_ew_unary(self.ctx, op, p, q, buf.len(), buf.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}
impl<Mods: OnDropBuffer + AddOperation + 'static, S: Shape> UnaryGrad<f32, S> for HIP<Mods> {
    fn add_unary_grad<F>(&self, lhs: &Buf<Mods, S>, lhs_grad: &mut Buf<Mods, S>, out: &Buf<Mods, S>, lhs_grad_fn: impl Fn(Resolve<f32>) -> F + Copy + 'static)
    where
        F: Eval<f32> + MayToCLSource,
    {
        let (op, p) = probe::unary_op_of_grad(lhs_grad_fn).expect("add_unary_grad: this derivative has no device kernel");
        check(unsafe { slhip_ew_unary_grad(self.ctx, op, p, lhs.len(), lhs.ptr(), lhs_grad.ptr_mut(), out.ptr()) }).unwrap();
    }
}

// ------------------------------------------------------------------------------------ diagflat, onehot
// src/ops2/diagflat/mod.rs, src/ops2/diagflat/grad.rs (x_grad[i] += out_grad[i*n + i])
impl<Mods: Retrieve<Self, f32> + 'static> Diagflat<f32> for HIP<Mods> {
    fn diagflat(&self, x: &Buf<Mods>) -> Buf<Mods> {
        let mut out = self.retrieve(x.len() * x.len(), x).unwrap();
        check(unsafe { slhip_diagflat(self.ctx, x.len(), x.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}
impl<Mods: OnDropBuffer + 'static> DiagflatGrad<f32> for HIP<Mods> {
    fn diagflat_grad(&self, x_grad: &mut Buf<Mods>, out_grad: &Buf<Mods>) {
        check(unsafe { slhip_diagflat_grad(self.ctx, x_grad.len(), x_grad.ptr_mut(), out_grad.ptr()) }).unwrap();
    }
}
// src/ops2/onehot/mod.rs: the class count is the largest class + 1 (src/ops2/onehot/cpu.rs:22-38)
impl<Mods: Retrieve<Self, f32> + 'static> Onehot<f32> for HIP<Mods> {
    fn onehot(&self, classes: &Buf<Mods>) -> Buf<Mods> {
        let highest = self.max(classes) as usize + 1;
        let mut out = self.retrieve(classes.len() * highest, classes).unwrap();
        check(unsafe { slhip_onehot(self.ctx, classes.len(), highest, classes.ptr(), out.ptr_mut()) }).unwrap();
        out
    }
}

// ------------------------------------------------------------------------------------ extras
/// Methods with no trait in the reference: fused forms of op chains its examples run, and the
/// host loops of the examples that a device-resident training loop needs as kernels.
impl<Mods: Retrieve<Self, f32> + 'static> HIP<Mods> {
    /// `gemm` + `add_row_mut` (+ `relu`) of examples/sine_net.rs:32-40 in one kernel.
    /// `pre_act` receives the value before the ReLU, which its gradient needs.
    pub fn linear(&self, m: usize, k: usize, n: usize, x: &Buf<Mods>, w: &Buf<Mods>, bias: &Buf<Mods>, relu: bool, pre_act: Option<&mut Buf<Mods>>) -> Buf<Mods> {
        let mut out = self.retrieve(m * n, (x, w)).unwrap();
        let pre = pre_act.map_or(core::ptr::null_mut(), |b| b.ptr_mut());
        check(unsafe { slhip_linear_fwd(self.ctx, m, k, n, x.ptr(), w.ptr(), bias.ptr(), relu as i32, pre, out.ptr_mut()) }).unwrap();
        out
    }
    /// The backward pass of that Linear: the gradients `gemm` (src/ops2/gemm/grad/cpu_stack.rs:36,39) and
    /// `add_row_mut` (src/ops2/row_op/grad/cpu.rs:42-50) leave on the tape, for small layers as one launch.
    /// `relu_pre`: pre-activations of the ReLU that produced `x`; its gradient is then taken on the way.
    #[allow(clippy::too_many_arguments)]
    pub fn linear_grad(&self, m: usize, k: usize, n: usize, x: &Buf<Mods>, w: &Buf<Mods>, x_grad: Option<&mut Buf<Mods>>, relu_pre: Option<&Buf<Mods>>, w_grad: Option<&mut Buf<Mods>>, bias_grad: Option<&mut Buf<Mods>>, out_grad: &Buf<Mods>) {
        let xg = x_grad.map_or(core::ptr::null_mut(), |b| b.ptr_mut());
        let wg = w_grad.map_or(core::ptr::null_mut(), |b| b.ptr_mut());
        let bg = bias_grad.map_or(core::ptr::null_mut(), |b| b.ptr_mut());
        let pre = relu_pre.map_or(core::ptr::null(), |b| b.ptr());
        check(unsafe { slhip_linear_grad(self.ctx, m, k, n, x.ptr(), w.ptr(), xg, pre, wg, bg, out_grad.ptr(), GRAD_BETA) }).unwrap();
    }
    /// `cce` of examples/nn.rs:124-138 on the device: loss[r] = -ln sum_c clip(p, 1e-7, 1 - 1e-7) * t.
    pub fn cce(&self, rows: usize, cols: usize, preds: &Buf<Mods>, targets: &Buf<Mods>) -> Buf<Mods> {
        let mut loss = self.retrieve(rows, (preds, targets)).unwrap();
        check(unsafe { slhip_cce(self.ctx, rows, cols, preds.ptr(), targets.ptr(), loss.ptr_mut()) }).unwrap();
        loss
    }
    /// `cce_grad` of examples/nn.rs:140-152: (-(t / p)) / rows.
    pub fn cce_grad(&self, rows: usize, cols: usize, preds: &Buf<Mods>, targets: &Buf<Mods>) -> Buf<Mods> {
        let mut grad = self.retrieve(rows * cols, (preds, targets)).unwrap();
        check(unsafe { slhip_cce_grad(self.ctx, rows, cols, preds.ptr(), targets.ptr(), grad.ptr_mut()) }).unwrap();
        grad
    }
    /// A chain of elementwise ops as one launch (`slhip_ew_program`): `inputs` are up to four buffers
    /// of one length, `prog` up to eight instructions (see `ffi::SlhipEwInsn`).
    pub fn ew_program(&self, inputs: &[&Buf<Mods>], prog: &[SlhipEwInsn]) -> Buf<Mods> {
        let ptrs: Vec<*const f32> = inputs.iter().map(|b| b.ptr()).collect();
        let mut out = self.retrieve(inputs[0].len(), inputs[0]).unwrap();
        check(unsafe { slhip_ew_program(self.ctx, inputs[0].len(), ptrs.len(), ptrs.as_ptr(), prog.len(), prog.as_ptr(), out.ptr_mut()) })
            .unwrap();
        out
    }
}
