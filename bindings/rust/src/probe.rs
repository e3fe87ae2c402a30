//! The reference passes its elementwise ops around as closures over custos' expression DSL
//! (`|lhs, rhs| lhs.add(rhs)`, src/ops2/binary_ew/mod.rs:60-100).  Its CPU device evaluates the
//! closure per element; its OpenCL device calls it once with string markers and pastes the result
//! into kernel source (src/ops2/binary_ew/opencl.rs:41-50).  A closure cannot cross a C ABI, and
//! the library has a fixed op set, so this device calls the closure on a few probe values and
//! recognises which op of the set it is.  Anything else is refused with a panic that names the
//! limitation - never computed on the host.
use custos::{Eval, Resolve, ToVal};

use crate::ffi::*;

const PROBES: [(f32, f32); 4] = [(3.0, 5.0), (-2.0, 7.0), (0.5, -4.0), (-1.25, -0.75)];

fn same(a: f32, b: f32) -> bool {
    a == b || (a - b).abs() <= 1e-6 * b.abs().max(1.0)
}

/// Which of add / sub / mul / div a binary closure is.
pub fn binary_op<O: Eval<f32>>(f: impl Fn(Resolve<f32>, Resolve<f32>) -> O) -> Option<i32> {
    let at = |a: f32, b: f32| f(a.to_val(), b.to_val()).eval();
    let cands: [(i32, fn(f32, f32) -> f32); 4] =
        [(SLHIP_ADD, |a, b| a + b), (SLHIP_SUB, |a, b| a - b), (SLHIP_MUL, |a, b| a * b), (SLHIP_DIV, |a, b| a / b)];
    cands.iter().find(|(_, g)| PROBES.iter().all(|&(a, b)| same(at(a, b), g(a, b)))).map(|(op, _)| *op)
}

/// The op whose partial derivatives the pair of gradient closures computes
/// (`BinaryOpsMayGrad`, src/ops.rs:115-171: add (1, 1), sub (1, -1), mul (rhs, lhs)).
pub fn binary_op_of_grads<LO: Eval<f32>, RO: Eval<f32>>(
    lf: impl Fn(Resolve<f32>, Resolve<f32>) -> LO,
    rf: impl Fn(Resolve<f32>, Resolve<f32>) -> RO,
) -> Option<i32> {
    let l = |a: f32, b: f32| lf(a.to_val(), b.to_val()).eval();
    let r = |a: f32, b: f32| rf(a.to_val(), b.to_val()).eval();
    type D = fn(f32, f32) -> f32;
    let cands: [(i32, D, D); 4] = [
        (SLHIP_ADD, |_, _| 1.0, |_, _| 1.0),
        (SLHIP_SUB, |_, _| 1.0, |_, _| -1.0),
        (SLHIP_MUL, |_, b| b, |a, _| a),
        (SLHIP_DIV, |_, b| 1.0 / b, |a, b| -a / (b * b)),
    ];
    cands
        .iter()
        .find(|(_, dl, dr)| PROBES.iter().all(|&(a, b)| same(l(a, b), dl(a, b)) && same(r(a, b), dr(a, b))))
        .map(|(op, _, _)| *op)
}

/// A unary closure of `apply_fn` as (op code, p, q).  Recognised: square, relu (`geq(0) * x`),
/// exp, tanh, sigmoid, negated ln, scaling by a constant, clip to constants, and pow with a
/// constant exponent (the exponent is read off one probe and checked on the others).
pub fn unary_op<O: Eval<f32>>(f: impl Fn(Resolve<f32>) -> O) -> Option<(i32, f32, f32)> {
    let at = |x: f32| f(x.to_val()).eval();
    let xs = [0.75f32, 2.0, 3.5, -1.5];
    let fits = |g: &dyn Fn(f32) -> f32, xs: &[f32]| xs.iter().all(|&x| same(at(x), g(x)));
    if fits(&|x| x * x, &xs) {
        return Some((SLHIP_SQUARE, 0.0, 0.0));
    }
    if fits(&|x| if x >= 0.0 { x } else { 0.0 }, &xs) {
        return Some((SLHIP_RELU, 0.0, 0.0));
    }
    if fits(&|x| x.exp(), &xs) {
        return Some((SLHIP_EXP, 0.0, 0.0));
    }
    if fits(&|x| x.tanh(), &xs) {
        return Some((SLHIP_TANH, 0.0, 0.0));
    }
    if fits(&|x| 1.0 / (1.0 + (-x).exp()), &xs) {
        return Some((SLHIP_SIGMOID, 0.0, 0.0));
    }
    if fits(&|x| -x.ln(), &xs[..3]) {
        return Some((SLHIP_NEG_LN, 0.0, 0.0));
    }
    let k = at(1.0);
    if fits(&|x| x * k, &xs) {
        return Some((SLHIP_SCALE, k, 0.0));
    }
    let (lo, hi) = (at(-1.0e30), at(1.0e30));
    if lo < hi && fits(&|x| x.max(lo).min(hi), &[lo - 1.0, 0.5 * (lo + hi), hi + 1.0]) {
        return Some((SLHIP_CLIP, lo, hi));
    }
    let p = at(2.0).ln() / 2.0f32.ln();
    if p.is_finite() && fits(&|x| x.powf(p), &xs[..3]) {
        return Some((SLHIP_POW, p, 0.0));
    }
    None
}

/// The op whose derivative a gradient closure of `add_unary_grad` computes, given the forward op is
/// not known at that point (src/ops.rs:38-41: `x.mul(two)` for square; :67-72: `x.pow(rhs - 1).mul(rhs)`).
pub fn unary_op_of_grad<O: Eval<f32>>(f: impl Fn(Resolve<f32>) -> O) -> Option<(i32, f32)> {
    let at = |x: f32| f(x.to_val()).eval();
    let xs = [0.75f32, 2.0, 3.5];
    let fits = |g: &dyn Fn(f32) -> f32| xs.iter().all(|&x| same(at(x), g(x)));
    if fits(&|x| 2.0 * x) {
        return Some((SLHIP_SQUARE, 0.0));
    }
    if fits(&|x| x.exp()) {
        return Some((SLHIP_EXP, 0.0));
    }
    if fits(&|x| 1.0 - x.tanh() * x.tanh()) {
        return Some((SLHIP_TANH, 0.0));
    }
    if fits(&|x| {
        let e = (-x).exp();
        e / ((1.0 + e) * (1.0 + e))
    }) {
        return Some((SLHIP_SIGMOID, 0.0));
    }
    if same(at(-1.0), 0.0) && fits(&|_| 1.0) {
        return Some((SLHIP_RELU, 0.0));
    }
    let k = at(1.0);
    if fits(&|_| k) {
        return Some((SLHIP_SCALE, k));
    }
    // p * x^(p-1): at x = 1 the value is p
    if fits(&|x| k * x.powf(k - 1.0)) {
        return Some((SLHIP_POW, k));
    }
    None
}
