//! `Device` and `Buffer<T>` over the C ABI, shaped like the `krnl` types autograph's tensors hold
//! (`krnl::device::Device`, `krnl::buffer::{Buffer, Slice, SliceMut}`), plus the launch wrappers the
//! `#[cfg(feature = "device")]` branches of the dense-contraction path call instead of building and
//! dispatching a krnl kernel.  Source only: written without a Rust toolchain at hand, never compiled.
//!
//! Call sites in autograph (paths relative to its checkout):
//! * `fn gemm`, src/tensor/linalg.rs:281-353            -> [`gemm`]
//! * `im2col_conv2`, src/tensor/ops.rs:842-880           -> [`im2col_conv2`]
//! * `col2im_conv2`, src/tensor/ops.rs:992-1030          -> [`col2im_conv2`]
//! * `max_pool2` / `max_pool2_backward`, :1117-1133, :1252-1264 -> [`max_pool2`], [`max_pool2_backward`]
use std::{ffi::CStr, marker::PhantomData, os::raw::c_void};

use anyhow::{bail, Result};
use autograph_hip_sys as sys;
use half::bf16;

/// Turns a status code into `anyhow::Result`, with the library's own message.
pub fn check(code: i32) -> Result<()> {
    if code == sys::AGH_OK {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(sys::agh_last_error_string()) }.to_string_lossy().into_owned();
    bail!("autograph_hip [{code}]: {msg}")
}

/// The element types the path supports; `DTYPE` selects the `_f32` / `_bf16` entry point.
pub trait Scalar: Copy + 'static {
    const IS_BF16: bool;
}
impl Scalar for f32 {
    const IS_BF16: bool = false;
}
impl Scalar for bf16 {
    const IS_BF16: bool = true;
}

/// One GPU, one in-order stream (krnl's per-device queue).
#[derive(Clone, Debug, PartialEq, Eq)]
pub struct Device {
    index: i32,
}

impl Device {
    pub fn new(index: usize) -> Result<Self> {
        check(unsafe { sys::agh_init(index as i32) })?;
        Ok(Self { index: index as i32 })
    }
    pub fn index(&self) -> usize {
        self.index as usize
    }
    /// `device.wait()`
    pub fn wait(&self) -> Result<()> {
        check(unsafe { sys::agh_sync() })
    }
}

/// Owning device allocation, freed on drop (krnl `Buffer<T>`).
pub struct Buffer<T> {
    ptr: *mut c_void,
    len: usize,
    _m: PhantomData<T>,
}
unsafe impl<T: Send> Send for Buffer<T> {}
unsafe impl<T: Sync> Sync for Buffer<T> {}

impl<T: Copy> Buffer<T> {
    /// # Safety
    /// The contents are uninitialised, as with `Buffer::uninit` in krnl.
    pub unsafe fn uninit(_device: &Device, len: usize) -> Result<Self> {
        let mut ptr = std::ptr::null_mut();
        check(sys::agh_malloc(&mut ptr, len.max(1) * std::mem::size_of::<T>()))?;
        Ok(Self { ptr, len, _m: PhantomData })
    }
    pub fn from_slice(device: &Device, data: &[T]) -> Result<Self> {
        let out = unsafe { Self::uninit(device, data.len())? };
        check(unsafe { sys::agh_memcpy_h2d(out.ptr, data.as_ptr() as *const c_void, std::mem::size_of_val(data)) })?;
        check(unsafe { sys::agh_sync() })?;
        Ok(out)
    }
    /// `into_vec()`: blocking copy back
    pub fn to_vec(&self) -> Result<Vec<T>> {
        let mut v = Vec::<T>::with_capacity(self.len);
        check(unsafe { sys::agh_memcpy_d2h(v.as_mut_ptr() as *mut c_void, self.ptr, self.len * std::mem::size_of::<T>()) })?;
        unsafe { v.set_len(self.len) };
        Ok(v)
    }
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn as_ptr(&self) -> *const c_void {
        self.ptr
    }
    pub fn as_mut_ptr(&mut self) -> *mut c_void {
        self.ptr
    }
}

impl<T> Drop for Buffer<T> {
    fn drop(&mut self) {
        unsafe { sys::agh_free(self.ptr) };
    }
}

/// A strided 2-D view as `fn gemm` extracts it: buffer, element offset, row and column stride in
/// elements (signed), exactly the tuple of src/tensor/linalg.rs:285-299.
#[derive(Clone, Copy)]
pub struct MatrixView {
    pub ptr: *const c_void,
    pub offset: i64,
    pub rs: i64,
    pub cs: i64,
}

/// `C = alpha * A * B + beta * C` (src/tensor/linalg.rs:249-360).  Shape and type checks stay in
/// autograph (`bail!`s at :256-279); split-K is internal to the library.
#[allow(clippy::too_many_arguments)]
pub fn gemm<T: Scalar>(m: usize, k: usize, n: usize, alpha: f32, a: MatrixView, b: MatrixView, beta: f32, c_ptr: *mut c_void, c: MatrixView) -> Result<()> {
    let (m, k, n) = (m as i64, k as i64, n as i64);
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_gemm_bf16(m, k, n, alpha, a.ptr, a.offset, a.rs, a.cs, b.ptr, b.offset, b.rs, b.cs, beta, c_ptr, c.offset, c.rs, c.cs)
        } else {
            sys::agh_gemm_f32(m, k, n, alpha, a.ptr, a.offset, a.rs, a.cs, b.ptr, b.offset, b.rs, b.cs, beta, c_ptr, c.offset, c.rs, c.cs)
        }
    })
}

/// A strided view of up to four dimensions (pad leading dimensions with 1 and stride 0): buffer, element offset,
/// signed element strides.  A stride of 0 on a source broadcasts it.
#[derive(Clone, Copy)]
pub struct View4 {
    pub ptr: *const c_void,
    pub offset: i64,
    pub strides: [i64; 4],
}

/// `y += alpha * x` on views, the device branch of `assign(BinaryOp::Add, alpha, x, y)` behind `scaled_add` and
/// `add_assign` (src/tensor/ops.rs:192-204, :245-255, :257-318): `x` already broadcast to `dims` by the caller
/// (`rhs.broadcast(self.raw_dim())`, :287-291), product and sum each rounded to `T`.
pub fn scaled_add<T: Scalar>(y_ptr: *mut c_void, y: View4, alpha: f32, x: View4, dims: [usize; 4]) -> Result<()> {
    let d = [dims[0] as i64, dims[1] as i64, dims[2] as i64, dims[3] as i64];
    let (sy, sx) = (y.strides, x.strides);
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_scaled_add_strided_bf16(y_ptr, y.offset, sy[0], sy[1], sy[2], sy[3], alpha, x.ptr, x.offset, sx[0], sx[1], sx[2], sx[3], d[0], d[1], d[2], d[3])
        } else {
            sys::agh_scaled_add_strided_f32(y_ptr, y.offset, sy[0], sy[1], sy[2], sy[3], alpha, x.ptr, x.offset, sx[0], sx[1], sx[2], sx[3], d[0], d[1], d[2], d[3])
        }
    })
}

/// `Accuracy::accuracy` device branch (src/learn/criterion.rs:101-118): writes the number of correct rows as one
/// `u32` to `correct` (device memory or pinned host memory); u8 targets.
pub fn accuracy<T: Scalar>(x: *const c_void, target_u8: *const c_void, batch_size: usize, classes: usize, correct: *mut c_void) -> Result<()> {
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_accuracy_bf16(x, target_u8, batch_size as i64, classes as i64, correct)
        } else {
            sys::agh_accuracy_f32(x, target_u8, batch_size as i64, classes as i64, correct)
        }
    })
}

/// Geometry of a 2-D convolution's patch extraction (`Im2ColConv2Options` / `Col2ImConv2Options`).
#[derive(Clone, Copy, Debug)]
pub struct ConvGeometry {
    pub bs: usize,
    pub c: usize,
    /// im2col: the image; col2im: the patch grid (`options.shape`)
    pub hw: [usize; 2],
    pub filter: [usize; 2],
    pub padding: [usize; 2],
    pub stride: [usize; 2],
    pub dilation: [usize; 2],
}

macro_rules! conv_call {
    ($f32:ident, $bf16:ident, $T:ty, $x:expr, $y:expr, $g:expr) => {{
        let g = $g;
        let a = [
            g.bs as i64, g.c as i64, g.hw[0] as i64, g.hw[1] as i64, g.filter[0] as i64, g.filter[1] as i64, g.padding[0] as i64,
            g.padding[1] as i64, g.stride[0] as i64, g.stride[1] as i64, g.dilation[0] as i64, g.dilation[1] as i64,
        ];
        check(unsafe {
            if <$T>::IS_BF16 {
                sys::$bf16($x, $y, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9], a[10], a[11])
            } else {
                sys::$f32($x, $y, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9], a[10], a[11])
            }
        })
    }};
}

/// src/tensor/ops.rs:842-880: `x` standard-layout `[bs, c, ih, iw]`, `y` `[bs*oh*ow, c*fh*fw]`.
pub fn im2col_conv2<T: Scalar>(x: *const c_void, y: *mut c_void, g: &ConvGeometry) -> Result<()> {
    conv_call!(agh_im2col_conv2_f32, agh_im2col_conv2_bf16, T, x, y, g)
}

/// src/tensor/ops.rs:992-1030: `x` `[bs*ih*iw, c*fh*fw]`, `y` `[bs, c, oh, ow]`, host accumulation order.
pub fn col2im_conv2<T: Scalar>(x: *const c_void, y: *mut c_void, g: &ConvGeometry) -> Result<()> {
    conv_call!(agh_col2im_conv2_f32, agh_col2im_conv2_bf16, T, x, y, g)
}

/// src/tensor/ops.rs:1117-1133
pub fn max_pool2<T: Scalar>(x: *const c_void, y: *mut c_void, bc: usize, hw: [usize; 2], size: [usize; 2], strides: [usize; 2]) -> Result<()> {
    let a = [bc as i64, hw[0] as i64, hw[1] as i64, size[0] as i64, size[1] as i64, strides[0] as i64, strides[1] as i64];
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_max_pool2_bf16(x, y, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        } else {
            sys::agh_max_pool2_f32(x, y, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        }
    })
}

/// src/tensor/ops.rs:1252-1264: `dx` holds `x` on entry.
pub fn max_pool2_backward<T: Scalar>(dx: *mut c_void, dy: *const c_void, bc: usize, hw: [usize; 2], size: [usize; 2], strides: [usize; 2]) -> Result<()> {
    let a = [bc as i64, hw[0] as i64, hw[1] as i64, size[0] as i64, size[1] as i64, strides[0] as i64, strides[1] as i64];
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_max_pool2_backward_bf16(dx, dy, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        } else {
            sys::agh_max_pool2_backward_f32(dx, dy, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        }
    })
}

/// `Relu` then `MaxPool2` (layer.rs:1253-1267, :1193-1216) in one launch; bit-identical to the two calls.
pub fn relu_max_pool2<T: Scalar>(x: *const c_void, y: *mut c_void, bc: usize, hw: [usize; 2], size: [usize; 2], strides: [usize; 2]) -> Result<()> {
    let a = [bc as i64, hw[0] as i64, hw[1] as i64, size[0] as i64, size[1] as i64, strides[0] as i64, strides[1] as i64];
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_relu_max_pool2_bf16(x, y, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        } else {
            sys::agh_relu_max_pool2_f32(x, y, a[0], a[1], a[2], a[3], a[4], a[5], a[6])
        }
    })
}

/// The backward edges of that pair (layer.rs:205-220, :1542-1565) in one launch, from the relu's input `x`;
/// `nhwc` writes `dx` as the `[bs*ih*iw, c]` matrix of autograd.rs:429-445.  Windows must not overlap.
#[allow(clippy::too_many_arguments)]
pub fn max_pool2_relu_backward<T: Scalar>(x: *const c_void, dy: *const c_void, dx: *mut c_void, bs: usize, c: usize, hw: [usize; 2], size: [usize; 2], strides: [usize; 2], nhwc: bool) -> Result<()> {
    let a = [bs as i64, c as i64, hw[0] as i64, hw[1] as i64, size[0] as i64, size[1] as i64, strides[0] as i64, strides[1] as i64];
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_max_pool2_relu_backward_bf16(x, dy, dx, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], nhwc as i32)
        } else {
            sys::agh_max_pool2_relu_backward_f32(x, dy, dx, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], nhwc as i32)
        }
    })
}

/// The input-gradient edge of `conv2_im2col` (layer.rs:976-988): `output_grad.dot(&weight_matrix)` and
/// `col2im_conv2` in one launch.  `g.hw` is the patch grid; an `Err` carrying `AGH_ERANGE` means the filter bank
/// does not fit in LDS: call `gemm` and `col2im_conv2` instead.
pub fn conv2_backward_input<T: Scalar>(dy: *const c_void, w: *const c_void, dx: *mut c_void, outputs: usize, g: &ConvGeometry) -> Result<()> {
    let a = [
        g.bs as i64, g.c as i64, g.hw[0] as i64, g.hw[1] as i64, outputs as i64, g.filter[0] as i64, g.filter[1] as i64,
        g.padding[0] as i64, g.padding[1] as i64, g.stride[0] as i64, g.stride[1] as i64, g.dilation[0] as i64, g.dilation[1] as i64,
    ];
    check(unsafe {
        if T::IS_BF16 {
            sys::agh_conv2_backward_input_bf16(dy, w, dx, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9], a[10], a[11], a[12])
        } else {
            sys::agh_conv2_backward_input_f32(dy, w, dx, a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9], a[10], a[11], a[12])
        }
    })
}

/// Runs `f` with the library's second stream current: what `f` launches starts after everything launched
/// before and runs beside what is launched next, until `join`.  The two sides must write disjoint memory.
pub fn branch<R>(f: impl FnOnce() -> Result<R>) -> Result<R> {
    check(unsafe { sys::agh_branch_begin() })?;
    let out = f();
    check(unsafe { sys::agh_branch_end() })?;
    out
}

/// Later launches wait for every `branch` issued so far.
pub fn join() -> Result<()> {
    check(unsafe { sys::agh_branch_join() })
}
