// hip_device.rs -- the `Hip` device of zenu-matrix: `zenu-matrix/src/device/hip/mod.rs` of a
// build with the cargo feature `hip`.
//
// It takes the place of `device/nvidia/mod.rs:8-69` (DeviceBase) and of the `impl ... for Nvidia`
// blocks next to every operation trait (`operation/basic_operations.rs:186-229,424-438,488-560`,
// `operation/{asum,clip,copy_from,max,relu}.rs`, `nn/conv/nvidia.rs:124-155`).  Everything goes
// through the C ABI declared in `zenu_hip_sys.rs` (generated from include/zenu_hip.h); nothing
// here computes.  Written against the reference's trait signatures; never compiled in this
// repository (its image has no Rust toolchain) -- tests/test_rust_device.py checks, as text, that
// every method of every trait the `Device` bound requires outside `nn` is implemented here and
// that every foreign function called here is declared in zenu_hip_sys.rs.
//
// What stays outside this file, as for `Nvidia`: `Gemm` (BLAS: rocBLAS takes cuBLAS's place) and
// the `nn` traits BatchNormalization, ConvFwd, ConvBkwdData, ConvBkwdFilter, Pool2dImpl, Dropout
// (MIOpen takes cuDNN's place).  `ConvBias` is implemented here because its two kernels are part of
// zenu-cuda-kernel-sys.
//
// Three layers:
//   1. DeviceBase and the leaf traits: one call per 1-D strided run, exactly what the reference's
//      host recursion (with_clousers.rs:180-223) asks a device for.  With only this layer the
//      unchanged zenu-matrix already runs on the GPU, one launch per row.
//   2. NdOps: whole-view entry points.  A Matrix-level method asks the device first
//      (`D::binary_nd(..)`) and falls back to the recursion when the device declines (the default,
//      which `Cpu` and `Nvidia` keep).  `Hip` answers every one of them with ONE launch.
//   3. FusedUpdate: the optimizers' per-tensor operator chains as one launch per `update`.
use std::any::TypeId;
use std::cell::Cell;
use std::os::raw::{c_int, c_void};

use serde::{Deserialize, Serialize};

use zenu_hip_sys::*;

use crate::{
    device::{cpu::Cpu, Device, DeviceBase},
    dim::{DimDyn, DimTrait},
    matrix::{Matrix, Ref, Repr},
    memory_pool::MemPoolError,
    nn::conv::interface::ConvBias,
    num::Num,
    operation::{
        asum::Asum,
        basic_operations::{
            AbsOps, AcosOps, AddOps, AsinOps, AtanOps, CosOps, CoshOps, DivOps, ExpOps, LogOps,
            MulOps, PowOws, SinOps, SinhOps, SqrtOps, SubOps, TanOps, TanhOps,
        },
        clip::ClipOps,
        copy_from::CopyBlas,
        max::MaxIdx,
        relu::ReluOps,
    },
};

#[derive(Copy, Clone, Default, Debug, Serialize, Deserialize)]
pub struct Hip;

thread_local! {
    // the stream this thread's launches go to; null = the HIP null stream (the reference launches
    // everything on the CUDA null stream: zenu-cuda/src/kernel/mod.rs passes no stream at all)
    static STREAM: Cell<ZenuStream> = Cell::new(std::ptr::null_mut());
}

/// The stream this thread launches on.
#[must_use]
pub fn current_stream() -> ZenuStream {
    STREAM.with(Cell::get)
}

/// Make this thread launch on `stream` (created with `zenu_hip_stream_create`); returns the previous one.
pub fn set_current_stream(stream: ZenuStream) -> ZenuStream {
    STREAM.with(|s| s.replace(stream))
}

fn status_text(rc: c_int) -> String {
    let p = unsafe { zenu_hip_status_string(rc) };
    if p.is_null() {
        return format!("status {rc}");
    }
    unsafe { std::ffi::CStr::from_ptr(p) }.to_string_lossy().into_owned()
}

/// The reference panics where the library returns a status (shape / rank / axis): same messages.
fn ok(rc: c_int) {
    match rc {
        ZENU_OK => (),
        ZENU_ERR_RANK => panic!("The rank of the matrix is different."),
        ZENU_ERR_SHAPE => panic!("shape mismatch / shapes are not broadcast compatible"),
        ZENU_ERR_AXIS => panic!("Invalid axis"),
        _ => panic!("zenu_hip: {}", status_text(rc)),
    }
}

fn dtype<T: Num>() -> c_int {
    if TypeId::of::<T>() == TypeId::of::<f32>() {
        ZENU_F32
    } else if TypeId::of::<T>() == TypeId::of::<f64>() {
        ZENU_F64
    } else {
        unimplemented!("the tensor-kernel library holds f32 and f64 kernels")
    }
}

fn as_f64<T: Num>(x: T) -> f64 {
    x.to_f64().unwrap()
}

fn to_i64(n: usize) -> i64 {
    i64::try_from(n).unwrap()
}

/// A 1-D run of `n` elements `stride` apart: what every leaf method of the reference describes.
fn view1d<T>(ptr: *const T, n: usize, stride: usize) -> ZenuTensor {
    let mut t = ZenuTensor {
        ptr: ptr.cast_mut().cast::<c_void>(),
        ndim: 1,
        reserved: 0,
        shape: [0; ZENU_MAX_DIM],
        stride: [0; ZENU_MAX_DIM],
    };
    t.shape[0] = to_i64(n);
    t.stride[0] = to_i64(stride);
    t
}

/// A whole view: `as_ptr()` already includes the view's offset (matrix.rs:288-290).
fn desc<R: Repr, D: DeviceBase>(m: &Matrix<R, DimDyn, D>) -> ZenuTensor {
    let shape = m.shape();
    let stride = m.stride();
    let nd = shape.len();
    assert!(nd <= ZENU_MAX_DIM, "at most {ZENU_MAX_DIM} dimensions");
    let mut t = ZenuTensor {
        ptr: m.as_ptr().cast_mut().cast::<c_void>(),
        ndim: i32::try_from(nd).unwrap(),
        reserved: 0,
        shape: [0; ZENU_MAX_DIM],
        stride: [0; ZENU_MAX_DIM],
    };
    for i in 0..nd {
        t.shape[i] = to_i64(shape[i]);
        t.stride[i] = to_i64(stride[i]);
    }
    t
}

// ---- DeviceBase (device/mod.rs:33-69; Nvidia: device/nvidia/mod.rs:11-67) -----------------------------
//
// The caching allocator lives in the library (stream ordered, no synchronisation on a hit), so the
// memory-pool half of the trait forwards to it; ZENU_USE_MEMPOOL=0 is honoured inside the library.

impl DeviceBase for Hip {
    fn raw_drop_ptr<T>(ptr: *mut T) {
        ok(unsafe { zenu_hip_free(ptr.cast::<c_void>(), current_stream()) });
    }

    fn mem_pool_drop_ptr(ptr: *mut u8) -> Result<(), MemPoolError> {
        match unsafe { zenu_hip_free(ptr.cast::<c_void>(), current_stream()) } {
            ZENU_OK => Ok(()),
            _ => Err(MemPoolError::MemPoolFreeError),
        }
    }

    fn clone_ptr<T>(src: *const T, len: usize) -> *mut T {
        let bytes = len * std::mem::size_of::<T>();
        let dst = Self::alloc(bytes).unwrap().cast::<T>();
        ok(unsafe {
            zenu_hip_memcpy_d2d(dst.cast::<c_void>(), src.cast::<c_void>(), bytes, current_stream())
        });
        dst
    }

    fn assign_item<T: Num>(ptr: *mut T, offset: usize, value: T) {
        // one element, host to device (blocking, like the reference's set_memory kernel + sync)
        ok(unsafe {
            zenu_hip_memcpy_h2d(
                ptr.add(offset).cast::<c_void>(),
                std::ptr::addr_of!(value).cast::<c_void>(),
                std::mem::size_of::<T>(),
                current_stream(),
            )
        });
    }

    fn get_item<T: Num>(ptr: *const T, offset: usize) -> T {
        let mut value = T::zero();
        ok(unsafe {
            zenu_hip_memcpy_d2h(
                std::ptr::addr_of_mut!(value).cast::<c_void>(),
                ptr.add(offset).cast::<c_void>(),
                std::mem::size_of::<T>(),
                current_stream(),
            )
        });
        value
    }

    fn from_vec<T: Num>(vec: Vec<T>) -> *mut T {
        let bytes = vec.len() * std::mem::size_of::<T>();
        let ptr = Self::alloc(bytes).unwrap().cast::<T>();
        ok(unsafe {
            zenu_hip_memcpy_h2d(ptr.cast::<c_void>(), vec.as_ptr().cast::<c_void>(), bytes, current_stream())
        });
        ptr
    }

    fn zeros<T: Num>(len: usize) -> *mut T {
        // a fill kernel; the reference scales uninitialised memory by 0 (cublas_scal), which keeps NaN
        let bytes = len * std::mem::size_of::<T>();
        let ptr = Self::alloc(bytes).unwrap().cast::<T>();
        ok(unsafe { zenu_hip_memset_zero(ptr.cast::<c_void>(), bytes, current_stream()) });
        ptr
    }

    fn raw_alloc(num_bytes: usize) -> Result<*mut u8, String> {
        let mut p: *mut c_void = std::ptr::null_mut();
        match unsafe { zenu_hip_malloc(std::ptr::addr_of_mut!(p), num_bytes, current_stream()) } {
            ZENU_OK => Ok(p.cast::<u8>()),
            rc => Err(status_text(rc)),
        }
    }

    fn mem_pool_alloc(num_bytes: usize) -> Result<*mut u8, MemPoolError> {
        Self::raw_alloc(num_bytes).map_err(|_| MemPoolError::DeviceMallocError)
    }
}

impl Device for Hip {}

// ---- leaf traits: binary operators (basic_operations.rs:44-92) ----------------------------------------

macro_rules! impl_hip_basic_op {
    ($name:ident, $op:expr) => {
        impl $name for Hip {
            fn array_array<T: Num>(
                to: *mut T,
                lhs: *const T,
                rhs: *const T,
                num_elm: usize,
                to_stride: usize,
                lhs_stride: usize,
                rhs_stride: usize,
            ) {
                let (t, l, r) = (
                    view1d(to, num_elm, to_stride),
                    view1d(lhs, num_elm, lhs_stride),
                    view1d(rhs, num_elm, rhs_stride),
                );
                ok(unsafe { zenu_hip_binary($op, dtype::<T>(), &t, &l, &r, current_stream()) });
            }

            fn array_assign<T: Num>(
                to: *mut T,
                rhs: *const T,
                num_elm: usize,
                to_stride: usize,
                rhs_stride: usize,
            ) {
                let (t, r) = (view1d(to, num_elm, to_stride), view1d(rhs, num_elm, rhs_stride));
                ok(unsafe { zenu_hip_binary_assign($op, dtype::<T>(), &t, &r, current_stream()) });
            }

            fn scalar<T: Num>(
                to: *mut T,
                lhs: *const T,
                rhs: T,
                num_elm: usize,
                to_stride: usize,
                lhs_stride: usize,
            ) {
                let (t, l) = (view1d(to, num_elm, to_stride), view1d(lhs, num_elm, lhs_stride));
                ok(unsafe {
                    zenu_hip_binary_scalar($op, dtype::<T>(), &t, &l, as_f64(rhs), current_stream())
                });
            }

            fn scalar_assign<T: Num>(to: *mut T, rhs: T, num_elm: usize, to_stride: usize) {
                let t = view1d(to, num_elm, to_stride);
                ok(unsafe {
                    zenu_hip_binary_scalar_assign($op, dtype::<T>(), &t, as_f64(rhs), current_stream())
                });
            }

            fn scalar_ptr<T: Num>(
                to: *mut T,
                rhs: *const T,
                scalar: *const T,
                to_stride: usize,
                rhs_stride: usize,
                num_elm: usize,
            ) {
                let (t, r) = (view1d(to, num_elm, to_stride), view1d(rhs, num_elm, rhs_stride));
                ok(unsafe {
                    zenu_hip_binary_scalar_ptr(
                        $op,
                        dtype::<T>(),
                        &t,
                        &r,
                        scalar.cast::<c_void>(),
                        current_stream(),
                    )
                });
            }

            fn scalar_assign_ptr<T: Num>(to: *mut T, scalar: *const T, num_elm: usize, to_stride: usize) {
                let t = view1d(to, num_elm, to_stride);
                ok(unsafe {
                    zenu_hip_binary_scalar_assign_ptr(
                        $op,
                        dtype::<T>(),
                        &t,
                        scalar.cast::<c_void>(),
                        current_stream(),
                    )
                });
            }
        }
    };
}
impl_hip_basic_op!(AddOps, ZENU_ADD);
impl_hip_basic_op!(SubOps, ZENU_SUB);
impl_hip_basic_op!(MulOps, ZENU_MUL);
impl_hip_basic_op!(DivOps, ZENU_DIV);

// ---- leaf traits: unary functions (basic_operations.rs:383-451) ------------------------------------

macro_rules! impl_hip_unary_op {
    ($name:ident, $fn_code:expr) => {
        impl $name for Hip {
            fn array<T: Num>(
                to: *mut T,
                other: *const T,
                num_elm: usize,
                to_stride: usize,
                other_stride: usize,
            ) {
                let (t, o) = (view1d(to, num_elm, to_stride), view1d(other, num_elm, other_stride));
                ok(unsafe { zenu_hip_unary($fn_code, dtype::<T>(), &t, &o, current_stream()) });
            }

            fn array_assign<T: Num>(to: *mut T, num_elm: usize, to_stride: usize) {
                let t = view1d(to, num_elm, to_stride);
                ok(unsafe { zenu_hip_unary_assign($fn_code, dtype::<T>(), &t, current_stream()) });
            }
        }
    };
}
impl_hip_unary_op!(SinOps, ZENU_SIN);
impl_hip_unary_op!(CosOps, ZENU_COS);
impl_hip_unary_op!(TanOps, ZENU_TAN);
impl_hip_unary_op!(AsinOps, ZENU_ASIN);
impl_hip_unary_op!(AcosOps, ZENU_ACOS);
impl_hip_unary_op!(AtanOps, ZENU_ATAN);
impl_hip_unary_op!(SinhOps, ZENU_SINH);
impl_hip_unary_op!(CoshOps, ZENU_COSH);
impl_hip_unary_op!(TanhOps, ZENU_TANH);
impl_hip_unary_op!(AbsOps, ZENU_ABS);
impl_hip_unary_op!(SqrtOps, ZENU_SQRT);
impl_hip_unary_op!(ExpOps, ZENU_EXP);
impl_hip_unary_op!(LogOps, ZENU_LOG);

// basic_operations.rs:453-463
impl PowOws for Hip {
    fn array<T: Num>(
        to: *mut T,
        other: *const T,
        scalar: T,
        num_elm: usize,
        to_stride: usize,
        other_stride: usize,
    ) {
        let (t, o) = (view1d(to, num_elm, to_stride), view1d(other, num_elm, other_stride));
        ok(unsafe { zenu_hip_powf(dtype::<T>(), &t, &o, as_f64(scalar), current_stream()) });
    }

    fn array_assign<T: Num>(to: *mut T, scalar: T, num_elm: usize, to_stride: usize) {
        let t = view1d(to, num_elm, to_stride);
        ok(unsafe { zenu_hip_powf(dtype::<T>(), &t, &t, as_f64(scalar), current_stream()) });
    }
}

// ---- leaf traits: the rest ---------------------------------------------------------------------------

// copy_from.rs:9-11
impl CopyBlas for Hip {
    fn copy_raw<T: Num>(n: usize, x: *const T, incx: usize, y: *mut T, incy: usize) {
        let (src, dst) = (view1d(x, n, incx), view1d(y, n, incy));
        ok(unsafe { zenu_hip_copy(dtype::<T>(), &dst, &src, current_stream()) });
    }
}

// asum.rs:14-16: the sum of |x| comes back to the host, as from BLAS
impl Asum for Hip {
    fn asum<T: Num>(n: usize, x: *const T, incx: usize) -> T {
        let out = Self::alloc(std::mem::size_of::<T>()).unwrap().cast::<T>();
        let src = view1d(x, n, incx);
        ok(unsafe { zenu_hip_asum(dtype::<T>(), out.cast::<c_void>(), &src, current_stream()) });
        let value = Self::get_item(out, 0);
        Self::drop_ptr(out);
        value
    }
}

// max.rs:15-17: index of the first largest element (the library follows the CPU scan of max.rs:22-32,
// for any length)
impl MaxIdx for Hip {
    fn max_idx<T: Num>(input: *const T, size: usize, stride: usize) -> usize {
        let mut out: c_int = 0;
        let (n, s) = (c_int::try_from(size).unwrap(), c_int::try_from(stride).unwrap());
        if T::is_f32() {
            unsafe { array_max_idx_float(input.cast_mut().cast::<f32>(), n, s, std::ptr::addr_of_mut!(out)) };
        } else {
            unsafe { array_max_idx_double(input.cast_mut().cast::<f64>(), n, s, std::ptr::addr_of_mut!(out)) };
        }
        ok(unsafe { zenu_hip_last_status() });
        usize::try_from(out).unwrap()
    }
}

// relu.rs:12-29
impl ReluOps for Hip {
    fn relu<T: Num>(
        input: *const T,
        output: *mut T,
        alpha: T,
        size: usize,
        input_stride: usize,
        output_stride: usize,
    ) {
        let (o, i) = (view1d(output, size, output_stride), view1d(input, size, input_stride));
        ok(unsafe { zenu_hip_relu(dtype::<T>(), &o, &i, as_f64(alpha), current_stream()) });
    }

    fn relu_backward_mask<T: Num>(
        input: *const T,
        mask: *mut T,
        alpha: T,
        size: usize,
        input_stride: usize,
        mask_stride: usize,
    ) {
        let (m, i) = (view1d(mask, size, mask_stride), view1d(input, size, input_stride));
        ok(unsafe { zenu_hip_relu_backward_mask(dtype::<T>(), &m, &i, as_f64(alpha), current_stream()) });
    }
}

// clip.rs:15-36 (clip_backward: `max` comes before `min` in the trait, as in the CUDA kernel)
impl ClipOps for Hip {
    fn clip<T: Num>(
        input: *const T,
        output: *mut T,
        size: usize,
        stride_in: usize,
        stride_out: usize,
        min: T,
        max: T,
    ) {
        let (o, i) = (view1d(output, size, stride_out), view1d(input, size, stride_in));
        ok(unsafe { zenu_hip_clip(dtype::<T>(), &o, &i, as_f64(min), as_f64(max), current_stream()) });
    }

    fn clip_assign<T: Num>(input: *mut T, size: usize, stride: usize, min: T, max: T) {
        let t = view1d(input, size, stride);
        ok(unsafe { zenu_hip_clip(dtype::<T>(), &t, &t, as_f64(min), as_f64(max), current_stream()) });
    }

    fn clip_backward<T: Num>(
        input: *const T,
        mask: *mut T,
        max: T,
        min: T,
        size: usize,
        stride_in: usize,
        stride_out: usize,
    ) {
        let (m, i) = (view1d(mask, size, stride_out), view1d(input, size, stride_in));
        ok(unsafe {
            zenu_hip_clip_backward_mask(dtype::<T>(), &m, &i, as_f64(min), as_f64(max), current_stream())
        });
    }

    fn clip_backward_assign<T: Num>(mask: *mut T, max: T, min: T, size: usize, stride: usize) {
        let m = view1d(mask, size, stride);
        ok(unsafe {
            zenu_hip_clip_backward_mask(dtype::<T>(), &m, &m, as_f64(min), as_f64(max), current_stream())
        });
    }
}

// nn/conv/interface.rs:46-57, Nvidia: nn/conv/nvidia.rs:124-155 -- same two kernels, same arguments
impl ConvBias for Hip {
    fn conv2d_bias<T: Num>(
        input: Matrix<Ref<&T>, DimDyn, Self>,
        bias: Matrix<Ref<&T>, DimDyn, Self>,
        output: Matrix<Ref<&mut T>, DimDyn, Self>,
    ) {
        let channel_stride = c_int::try_from(input.stride()[1]).unwrap();
        let total = c_int::try_from(input.shape().num_elm()).unwrap();
        let bias_size = c_int::try_from(bias.shape().num_elm()).unwrap();
        if T::is_f32() {
            unsafe {
                conv_bias_add_float(
                    input.as_ptr().cast::<f32>(),
                    output.as_mut_ptr().cast::<f32>(),
                    channel_stride,
                    bias.as_ptr().cast::<f32>(),
                    bias_size,
                    total,
                );
            }
        } else {
            unsafe {
                conv_bias_add_double(
                    input.as_ptr().cast::<f64>(),
                    output.as_mut_ptr().cast::<f64>(),
                    channel_stride,
                    bias.as_ptr().cast::<f64>(),
                    bias_size,
                    total,
                );
            }
        }
        ok(unsafe { zenu_hip_last_status() });
    }

    fn conv2d_bias_bkwd<T: Num>(
        d_output: Matrix<Ref<&T>, DimDyn, Self>,
        bias: Matrix<Ref<&mut T>, DimDyn, Self>,
    ) {
        let dims: Vec<c_int> = (0..4).map(|i| c_int::try_from(d_output.shape()[i]).unwrap()).collect();
        if T::is_f32() {
            unsafe {
                conv2d_bias_bkwd_float(
                    d_output.as_ptr().cast::<f32>(),
                    bias.as_mut_ptr().cast::<f32>(),
                    dims[0],
                    dims[1],
                    dims[2],
                    dims[3],
                );
            }
        } else {
            unsafe {
                conv2d_bias_bkwd_double(
                    d_output.as_ptr().cast::<f64>(),
                    bias.as_mut_ptr().cast::<f64>(),
                    dims[0],
                    dims[1],
                    dims[2],
                    dims[3],
                );
            }
        }
        ok(unsafe { zenu_hip_last_status() });
    }
}

// ---- layer 2: whole views in one launch ----------------------------------------------------------------
//
// The reference resolves an N-d, strided or broadcast call by recursing over the leading axis on the
// host and calling a leaf method per row (with_clousers.rs:180-223): 4096 launches for
// a[4096,4096] + b[1,4096].  A device that can take the whole view says so by returning `true`;
// the Matrix-level method then skips its recursion:
//
//     // basic_operations.rs:336-356, `$method` of impl_basic_ops!
//     pub fn add_array<..>(&self, lhs, rhs) {
//         if D::binary_nd(BinaryOp::Add, self, &lhs.to_ref(), &rhs.to_ref()) { return; }
//         array_array_array(self, lhs, rhs, |..| D::array_array(..));      // as today
//     }
//
// `Cpu` (and `Nvidia`) keep the defaults, so nothing changes for them.

#[derive(Copy, Clone, Debug, PartialEq, Eq)]
pub enum BinaryOp {
    Add,
    Sub,
    Mul,
    Div,
}

impl BinaryOp {
    fn code(self) -> c_int {
        match self {
            BinaryOp::Add => ZENU_ADD,
            BinaryOp::Sub => ZENU_SUB,
            BinaryOp::Mul => ZENU_MUL,
            BinaryOp::Div => ZENU_DIV,
        }
    }
}

#[derive(Copy, Clone, Debug, PartialEq, Eq)]
pub enum UnaryFn {
    Exp,
    Log,
    Tanh,
    Sqrt,
    Abs,
    Sin,
    Cos,
    Tan,
    Asin,
    Acos,
    Atan,
    Sinh,
    Cosh,
    /// 0.5 + 0.5 tanh(0.5 x), rounded as the chain of zenu-autograd/src/activation/sigmoid.rs:7-15
    Sigmoid,
}

impl UnaryFn {
    fn code(self) -> c_int {
        match self {
            UnaryFn::Exp => ZENU_EXP,
            UnaryFn::Log => ZENU_LOG,
            UnaryFn::Tanh => ZENU_TANH,
            UnaryFn::Sqrt => ZENU_SQRT,
            UnaryFn::Abs => ZENU_ABS,
            UnaryFn::Sin => ZENU_SIN,
            UnaryFn::Cos => ZENU_COS,
            UnaryFn::Tan => ZENU_TAN,
            UnaryFn::Asin => ZENU_ASIN,
            UnaryFn::Acos => ZENU_ACOS,
            UnaryFn::Atan => ZENU_ATAN,
            UnaryFn::Sinh => ZENU_SINH,
            UnaryFn::Cosh => ZENU_COSH,
            UnaryFn::Sigmoid => ZENU_SIGMOID,
        }
    }
}

type MutView<'a, T, D> = Matrix<Ref<&'a mut T>, DimDyn, D>;
type View<'a, T, D> = Matrix<Ref<&'a T>, DimDyn, D>;

pub trait NdOps: DeviceBase {
    /// `to = lhs op rhs` with ZeNu's broadcasting (basic_operations.rs:336-356)
    fn binary_nd<T: Num>(_op: BinaryOp, _to: &MutView<T, Self>, _lhs: &View<T, Self>, _rhs: &View<T, Self>) -> bool {
        false
    }
    /// `to op= rhs` (basic_operations.rs:318-334)
    fn binary_assign_nd<T: Num>(_op: BinaryOp, _to: &MutView<T, Self>, _rhs: &View<T, Self>) -> bool {
        false
    }
    /// `to = other op scalar` (basic_operations.rs:291-308)
    fn scalar_nd<T: Num>(_op: BinaryOp, _to: &MutView<T, Self>, _other: &View<T, Self>, _scalar: T) -> bool {
        false
    }
    /// `to op= scalar` (basic_operations.rs:310-316)
    fn scalar_assign_nd<T: Num>(_op: BinaryOp, _to: &MutView<T, Self>, _scalar: T) -> bool {
        false
    }
    /// `to = f(other)` (basic_operations.rs:515-537)
    fn unary_nd<T: Num>(_f: UnaryFn, _to: &MutView<T, Self>, _other: &View<T, Self>) -> bool {
        false
    }
    /// `to = f(to)` (basic_operations.rs:539-553)
    fn unary_assign_nd<T: Num>(_f: UnaryFn, _to: &MutView<T, Self>) -> bool {
        false
    }
    /// relu.rs:171-204
    fn relu_nd<T: Num>(_to: &MutView<T, Self>, _other: &View<T, Self>, _alpha: T) -> bool {
        false
    }
    /// relu.rs:206-242
    fn relu_backward_mask_nd<T: Num>(_to: &MutView<T, Self>, _other: &View<T, Self>, _alpha: T) -> bool {
        false
    }
    /// copy_from.rs:263-267
    fn copy_nd<T: Num>(_to: &MutView<T, Self>, _src: &View<T, Self>) -> bool {
        false
    }
    /// broadcast.rs:11-43
    fn broadcast_nd<T: Num>(_to: &MutView<T, Self>, _source: &View<T, Self>) -> bool {
        false
    }
    /// sum.rs:12-31: `out` has the shape of `src` without `axis` (or with it kept as 1)
    fn sum_axis_nd<T: Num>(_out: &MutView<T, Self>, _src: &View<T, Self>, _axis: usize) -> bool {
        false
    }
    /// sum.rs:35-94
    fn sum_to_nd<T: Num>(_target: &MutView<T, Self>, _src: &View<T, Self>) -> bool {
        false
    }
    /// max.rs:67-99
    fn max_axis_nd<T: Num>(_out: &MutView<T, Self>, _src: &View<T, Self>, _axis: usize) -> bool {
        false
    }
    /// max.rs:103-135: the arg-max along `axis` of every line, in row-major order of the kept dims
    fn max_axis_idx_nd<T: Num>(_src: &View<T, Self>, _axis: usize) -> Option<Vec<usize>> {
        None
    }
    /// max.rs:45-57: the position of the largest element, as an index per dimension
    fn max_idx_nd<T: Num>(_src: &View<T, Self>) -> Option<Vec<usize>> {
        None
    }
    /// asum.rs:50-68
    fn asum_nd<T: Num>(_src: &View<T, Self>) -> Option<T> {
        None
    }
    /// softmax.rs:10-25
    fn softmax_nd<T: Num>(_to: &MutView<T, Self>, _source: &View<T, Self>, _axis: usize) -> bool {
        false
    }
    /// clip.rs:282-318
    fn clip_nd<T: Num>(_to: &MutView<T, Self>, _other: &View<T, Self>, _min: T, _max: T) -> bool {
        false
    }
}

impl NdOps for Cpu {}

#[cfg(feature = "nvidia")]
impl NdOps for crate::device::nvidia::Nvidia {}

impl NdOps for Hip {
    fn binary_nd<T: Num>(op: BinaryOp, to: &MutView<T, Self>, lhs: &View<T, Self>, rhs: &View<T, Self>) -> bool {
        ok(unsafe {
            zenu_hip_binary(op.code(), dtype::<T>(), &desc(to), &desc(lhs), &desc(rhs), current_stream())
        });
        true
    }

    fn binary_assign_nd<T: Num>(op: BinaryOp, to: &MutView<T, Self>, rhs: &View<T, Self>) -> bool {
        ok(unsafe { zenu_hip_binary_assign(op.code(), dtype::<T>(), &desc(to), &desc(rhs), current_stream()) });
        true
    }

    fn scalar_nd<T: Num>(op: BinaryOp, to: &MutView<T, Self>, other: &View<T, Self>, scalar: T) -> bool {
        ok(unsafe {
            zenu_hip_binary_scalar(op.code(), dtype::<T>(), &desc(to), &desc(other), as_f64(scalar), current_stream())
        });
        true
    }

    fn scalar_assign_nd<T: Num>(op: BinaryOp, to: &MutView<T, Self>, scalar: T) -> bool {
        ok(unsafe {
            zenu_hip_binary_scalar_assign(op.code(), dtype::<T>(), &desc(to), as_f64(scalar), current_stream())
        });
        true
    }

    fn unary_nd<T: Num>(f: UnaryFn, to: &MutView<T, Self>, other: &View<T, Self>) -> bool {
        ok(unsafe { zenu_hip_unary(f.code(), dtype::<T>(), &desc(to), &desc(other), current_stream()) });
        true
    }

    fn unary_assign_nd<T: Num>(f: UnaryFn, to: &MutView<T, Self>) -> bool {
        ok(unsafe { zenu_hip_unary_assign(f.code(), dtype::<T>(), &desc(to), current_stream()) });
        true
    }

    fn relu_nd<T: Num>(to: &MutView<T, Self>, other: &View<T, Self>, alpha: T) -> bool {
        ok(unsafe { zenu_hip_relu(dtype::<T>(), &desc(to), &desc(other), as_f64(alpha), current_stream()) });
        true
    }

    fn relu_backward_mask_nd<T: Num>(to: &MutView<T, Self>, other: &View<T, Self>, alpha: T) -> bool {
        ok(unsafe {
            zenu_hip_relu_backward_mask(dtype::<T>(), &desc(to), &desc(other), as_f64(alpha), current_stream())
        });
        true
    }

    fn copy_nd<T: Num>(to: &MutView<T, Self>, src: &View<T, Self>) -> bool {
        ok(unsafe { zenu_hip_copy(dtype::<T>(), &desc(to), &desc(src), current_stream()) });
        true
    }

    fn broadcast_nd<T: Num>(to: &MutView<T, Self>, source: &View<T, Self>) -> bool {
        ok(unsafe { zenu_hip_broadcast(dtype::<T>(), &desc(to), &desc(source), current_stream()) });
        true
    }

    fn sum_axis_nd<T: Num>(out: &MutView<T, Self>, src: &View<T, Self>, axis: usize) -> bool {
        let axis = c_int::try_from(axis).unwrap();
        ok(unsafe { zenu_hip_sum_axis(dtype::<T>(), &desc(out), &desc(src), axis, current_stream()) });
        true
    }

    fn sum_to_nd<T: Num>(target: &MutView<T, Self>, src: &View<T, Self>) -> bool {
        ok(unsafe { zenu_hip_sum_to(dtype::<T>(), &desc(target), &desc(src), current_stream()) });
        true
    }

    fn max_axis_nd<T: Num>(out: &MutView<T, Self>, src: &View<T, Self>, axis: usize) -> bool {
        let axis = c_int::try_from(axis).unwrap();
        ok(unsafe { zenu_hip_max_axis(dtype::<T>(), &desc(out), &desc(src), axis, current_stream()) });
        true
    }

    fn max_axis_idx_nd<T: Num>(src: &View<T, Self>, axis: usize) -> Option<Vec<usize>> {
        let lines = src.shape().num_elm() / src.shape()[axis].max(1);
        let bytes = lines * std::mem::size_of::<i64>();
        let dev = Self::alloc(bytes).unwrap().cast::<i64>();
        ok(unsafe {
            zenu_hip_max_axis_idx(dtype::<T>(), dev, &desc(src), c_int::try_from(axis).unwrap(), current_stream())
        });
        let mut host = vec![0_i64; lines];
        ok(unsafe {
            zenu_hip_memcpy_d2h(host.as_mut_ptr().cast::<c_void>(), dev.cast::<c_void>(), bytes, current_stream())
        });
        Self::drop_ptr(dev);
        Some(host.into_iter().map(|i| usize::try_from(i).unwrap()).collect())
    }

    fn max_idx_nd<T: Num>(src: &View<T, Self>) -> Option<Vec<usize>> {
        let dev = Self::alloc(std::mem::size_of::<i64>()).unwrap().cast::<i64>();
        ok(unsafe { zenu_hip_max_idx(dtype::<T>(), dev, std::ptr::null_mut(), &desc(src), current_stream()) });
        let mut flat = 0_i64;
        ok(unsafe {
            zenu_hip_memcpy_d2h(
                std::ptr::addr_of_mut!(flat).cast::<c_void>(),
                dev.cast::<c_void>(),
                std::mem::size_of::<i64>(),
                current_stream(),
            )
        });
        Self::drop_ptr(dev);
        // row-major position -> one index per dimension (max.rs:45-57)
        let shape = src.shape();
        let mut rest = usize::try_from(flat).unwrap();
        let mut index = vec![0_usize; shape.len()];
        for d in (0..shape.len()).rev() {
            index[d] = rest % shape[d];
            rest /= shape[d];
        }
        Some(index)
    }

    fn asum_nd<T: Num>(src: &View<T, Self>) -> Option<T> {
        let out = Self::alloc(std::mem::size_of::<T>()).unwrap().cast::<T>();
        ok(unsafe { zenu_hip_asum(dtype::<T>(), out.cast::<c_void>(), &desc(src), current_stream()) });
        let value = Self::get_item(out, 0);
        Self::drop_ptr(out);
        Some(value)
    }

    fn softmax_nd<T: Num>(to: &MutView<T, Self>, source: &View<T, Self>, axis: usize) -> bool {
        let axis = c_int::try_from(axis).unwrap();
        ok(unsafe { zenu_hip_softmax(dtype::<T>(), &desc(to), &desc(source), axis, current_stream()) });
        true
    }

    fn clip_nd<T: Num>(to: &MutView<T, Self>, other: &View<T, Self>, min: T, max: T) -> bool {
        ok(unsafe {
            zenu_hip_clip(dtype::<T>(), &desc(to), &desc(other), as_f64(min), as_f64(max), current_stream())
        });
        true
    }
}

// ---- layer 3: the optimizers' updates as one launch ----------------------------------------------------
//
// zenu-optimizer's `update` methods are generic over the device, so the device is asked, like
// above.  One tensor of an update: parameter, gradient and (for Adam) both moments, all default
// stride (they are whole tensors in the reference too), `len` elements each.
//
//     // zenu-optimizer/src/adam.rs:20-58
//     fn update(&self, parameters: &P) {
//         *self.step.borrow_mut() += 1;
//         let tensors = ...;        // (p, g, m, v) of every parameter that has a gradient
//         if D::adam_update(&tensors, lr, beta1, beta2, eps, T::zero(), None, step) { return; }
//         for (k, (data, grad)) in &parameters { ... }                     // as today
//     }

pub struct UpdateTensor<T> {
    pub param: *mut T,
    pub grad: *const T,
    pub m: *mut T,
    pub v: *mut T,
    pub len: usize,
}

pub trait FusedUpdate: DeviceBase {
    /// sgd.rs:20-31: `p -= g * lr` for every tensor
    fn sgd_update<T: Num>(_tensors: &[UpdateTensor<T>], _learning_rate: T) -> bool {
        false
    }
    /// adam.rs:19-59 (weight_decay = 0, decay = None) and adamw.rs:20-70 (`decay[i]` is true for the keys
    /// of `Parameters::weights()`); `step` is the counter after its increment
    #[allow(clippy::too_many_arguments)]
    fn adam_update<T: Num>(
        _tensors: &[UpdateTensor<T>],
        _learning_rate: T,
        _beta1: T,
        _beta2: T,
        _epsilon: T,
        _weight_decay: T,
        _decay: Option<&[bool]>,
        _step: usize,
    ) -> bool {
        false
    }
}

impl FusedUpdate for Cpu {}

#[cfg(feature = "nvidia")]
impl FusedUpdate for crate::device::nvidia::Nvidia {}

impl FusedUpdate for Hip {
    fn sgd_update<T: Num>(tensors: &[UpdateTensor<T>], learning_rate: T) -> bool {
        let p: Vec<*mut c_void> = tensors.iter().map(|t| t.param.cast::<c_void>()).collect();
        let g: Vec<*const c_void> = tensors.iter().map(|t| t.grad.cast::<c_void>()).collect();
        let n: Vec<i64> = tensors.iter().map(|t| to_i64(t.len)).collect();
        ok(unsafe {
            zenu_hip_sgd_step_multi(
                dtype::<T>(),
                c_int::try_from(tensors.len()).unwrap(),
                p.as_ptr(),
                g.as_ptr(),
                n.as_ptr(),
                as_f64(learning_rate),
                current_stream(),
            )
        });
        true
    }

    fn adam_update<T: Num>(
        tensors: &[UpdateTensor<T>],
        learning_rate: T,
        beta1: T,
        beta2: T,
        epsilon: T,
        weight_decay: T,
        decay: Option<&[bool]>,
        step: usize,
    ) -> bool {
        let p: Vec<*mut c_void> = tensors.iter().map(|t| t.param.cast::<c_void>()).collect();
        let g: Vec<*const c_void> = tensors.iter().map(|t| t.grad.cast::<c_void>()).collect();
        let m: Vec<*mut c_void> = tensors.iter().map(|t| t.m.cast::<c_void>()).collect();
        let v: Vec<*mut c_void> = tensors.iter().map(|t| t.v.cast::<c_void>()).collect();
        let n: Vec<i64> = tensors.iter().map(|t| to_i64(t.len)).collect();
        let flags: Option<Vec<i32>> = decay.map(|d| d.iter().map(|&b| i32::from(b)).collect());
        let flags_ptr = flags.as_ref().map_or(std::ptr::null(), |f| f.as_ptr());
        // 1 - beta, beta^step and 1 - beta^step are formed inside the call, on the host, in T, with
        // libm's powf / pow -- the operations of adam.rs:22-25,45-51
        ok(unsafe {
            zenu_hip_adam_step_multi(
                dtype::<T>(),
                c_int::try_from(tensors.len()).unwrap(),
                p.as_ptr(),
                g.as_ptr(),
                m.as_ptr(),
                v.as_ptr(),
                n.as_ptr(),
                as_f64(learning_rate),
                as_f64(beta1),
                as_f64(beta2),
                as_f64(epsilon),
                as_f64(weight_decay),
                flags_ptr,
                step as f64,
                current_stream(),
            )
        });
        true
    }
}

// ---- host <-> device (matrix.rs:139-160, Ptr::to) --------------------------------------------------------

/// Device copy of a host buffer: what `Ptr<_, Cpu>::to::<Hip>()` calls.
pub fn upload<T: Num>(host: *const T, len: usize) -> *mut T {
    let bytes = len * std::mem::size_of::<T>();
    let dev = Hip::alloc(bytes).unwrap().cast::<T>();
    ok(unsafe { zenu_hip_memcpy_h2d(dev.cast::<c_void>(), host.cast::<c_void>(), bytes, current_stream()) });
    dev
}

/// Host copy of a device buffer into `host` (`len` elements): what `Ptr<_, Hip>::to::<Cpu>()` calls.
pub fn download<T: Num>(host: *mut T, dev: *const T, len: usize) {
    let bytes = len * std::mem::size_of::<T>();
    ok(unsafe { zenu_hip_memcpy_d2h(host.cast::<c_void>(), dev.cast::<c_void>(), bytes, current_stream()) });
}

/// Call once before the first allocation (the reference initialises its pool lazily through
/// ZENU_MATRIX_STATE, lib.rs:30-50; the library does the same on first use, this only picks the device).
pub fn init(device: i32) {
    ok(unsafe { zenu_hip_init(device) });
}

/// Optional start-up check of the one thing the bit-exact f32 functions take on trust from the GPU
/// they run on: `tanh`, the sigmoid, `sinh`, `cosh`, `tan`, `atan`, `asin` and `acos` divide (and take square
/// roots) with a short device sequence that is only correct on their own operand ranges.  The library
/// evaluates each function with that sequence and with the IEEE operations on all 2^32 arguments
/// (10-80 ms per function) and counts the arguments whose results differ; anything but zero is an error.
pub fn self_check() -> Result<(), String> {
    const FUNCTIONS: [(c_int, &str); 8] = [
        (ZENU_TANH, "tanh"),
        (ZENU_SIGMOID, "sigmoid"),
        (ZENU_SINH, "sinh"),
        (ZENU_COSH, "cosh"),
        (ZENU_TAN, "tan"),
        (ZENU_ATAN, "atan"),
        (ZENU_ASIN, "asin"),
        (ZENU_ACOS, "acos"),
    ];
    for (function, name) in FUNCTIONS {
        let mut mismatches: u64 = 0;
        let mut example: u32 = 0;
        ok(unsafe { zenu_hip_selfcheck_short_division(function, &mut mismatches, &mut example, current_stream()) });
        if mismatches != 0 {
            return Err(format!(
                "{name}: {mismatches} of 2^32 f32 arguments differ between the short and the IEEE division, e.g. bits {example:#010x}"
            ));
        }
    }
    Ok(())
}

/// Does the host libm behind the `Cpu` device give, for `function` (a `ZENU_*` unary id), the bits this device
/// gives?  Both sides fold their results over the f32 bit patterns `first .. first + count` (count a
/// multiple of 2^20) into one 64-bit sum per 2^20 arguments -- the device in `zenu_hip_unary_range_hash`,
/// the host here with `host` (e.g. `f32::tanh`; for `ZENU_SIGMOID` the composite
/// `|x| 0.5 + 0.5 * (x * 0.5).tanh()`) -- and the sums are compared: equal sums, equal bits on every
/// argument, and no result crosses the bus.  All 2^32 arguments take the device 0.1 s and one host
/// thread about half a minute; split the range over threads for less.
pub fn agrees_with_host_libm(function: c_int, host: fn(f32) -> f32, first: u64, count: u64) -> bool {
    const BLOCK_LOG2: c_int = 20;
    let blocks = (count >> BLOCK_LOG2) as usize;
    let bytes = blocks * std::mem::size_of::<u64>();
    let dev = Hip::alloc(bytes).unwrap();
    ok(unsafe { zenu_hip_unary_range_hash(function, first, count, BLOCK_LOG2, dev.cast::<u64>(), current_stream()) });
    let mut device_sums = vec![0u64; blocks];
    ok(unsafe { zenu_hip_memcpy_d2h(device_sums.as_mut_ptr().cast::<c_void>(), dev.cast::<c_void>(), bytes, current_stream()) });
    Hip::drop_ptr(dev);
    let mix = |mut z: u64| {
        z = (z ^ (z >> 30)).wrapping_mul(0xbf58_476d_1ce4_e5b9);
        z = (z ^ (z >> 27)).wrapping_mul(0x94d0_49bb_1331_11eb);
        z ^ (z >> 31)
    };
    for (b, device_sum) in device_sums.iter().enumerate() {
        let start = first + ((b as u64) << BLOCK_LOG2);
        let mut sum = 0u64;
        let mut offset = 0u64;
        while offset < (1u64 << BLOCK_LOG2) {
            let bits = (start + offset) as u32;
            offset += 1;
            let mut result = host(f32::from_bits(bits)).to_bits();
            if result & 0x7fff_ffff > 0x7f80_0000 {
                result = 0x7fc0_0000; // every NaN counts as one value
            }
            sum = sum.wrapping_add(mix((u64::from(bits) << 32) | u64::from(result)));
        }
        if sum != *device_sum {
            return false;
        }
    }
    true
}
