//! `Hip` device and `HipBackend`: rai's primitives evaluated by librai_hip.so on AMD MI355X.
//!
//! Drop-in sibling of `backend/candle.rs`: the storage type (`HipData`, a ref-counted strided view of device
//! memory) implements `TensorLike` (tensor.rs:19-26), and there is one `impl Eval<Hip, ops::X> for HipBackend`
//! per primitive that `register_backend!` lists (dispatch.rs:41-157) and that has a HIP kernel.  Ops without one
//! (Random, Normal, the convolution / pooling / upsampling family) are left unregistered, so evaluating them on
//! `Hip` yields `Error::Unimplemented { op, device }` from eval.rs:40-43 exactly as for any other missing rule.
//!
//! To add to a rai 0.11 checkout (not compiled in the repository this file ships in: no Rust toolchain there):
//!   * `rai-core/Cargo.toml`: `[features] hip = []`, `build = "build.rs"`;
//!   * `rai-core/src/backend/mod.rs`: `#[cfg(feature = "hip")] mod hip_sys; #[cfg(feature = "hip")] mod hip;
//!     #[cfg(feature = "hip")] pub use hip::{Hip, HipBackend, HipData, hip_if_available};`
//!   * `rai-core/src/lib.rs`: re-export `Hip`, `HipBackend` next to `Cuda`, `CandleBackend`;
//!   * `rai-core/src/dispatch.rs`, inside the `EVAL_DISPATCHER` initialiser after the Cuda/Metal lines (:166-169):
//!     `#[cfg(feature = "hip")] crate::backend::hip::register_hip(&mut rules);` with `_register` and the
//!     `DynBackend` alias made `pub(crate)`.
//! After that `Tensor::ones([2, 3], F32, Hip::new(0))`, `eval`, `grad` / `vjp` graphs, rai-nn modules and the
//! rai-models LLMs run unchanged: they only build graphs of these primitives.
use super::hip_sys::*;
use crate::{
    dispatch::DynBackend, ops, tensor::TensorLike, Backend, CandleBackend, Cpu, DType, Device, Eval, FloatElemType, Op,
    Tensor, Type, BF16, F16, F32, F64, I64, U32, U8,
};
use half::{bf16, f16};
use std::{
    any::{Any, TypeId},
    borrow::Cow,
    collections::HashMap,
    ffi::{c_int, c_void},
    fmt::{Debug, Display},
    ops::Deref,
};

// ------------------------------------------------------------------------------------------------ device
/// AMD GPU `id` driven through HIP.  Sibling of `Cuda(usize)` (device.rs:161-196).
#[derive(Debug, Clone, Copy, PartialEq, Eq, Hash)]
pub struct Hip(usize);

impl Hip {
    pub fn new(id: usize) -> Self {
        Self(id)
    }

    pub fn id(&self) -> usize {
        self.0
    }

    #[inline]
    fn dev(&self) -> c_int {
        self.0 as c_int
    }
}

impl Device for Hip {
    fn name(&self) -> Cow<'static, str> {
        Cow::Borrowed("hip")
    }

    fn as_any(&self) -> &dyn Any {
        self
    }

    fn clone_boxed(&self) -> Box<dyn Device> {
        Box::new(*self)
    }

    fn eq(&self, rhs: &dyn Device) -> bool {
        rhs.as_any().downcast_ref::<Self>().map_or(false, |other| self == other)
    }

    fn to_device_op(&self) -> Box<dyn Op> {
        Box::new(ops::ToDevice::new(*self))
    }
}

/// `cuda_if_available` (device.rs:198-204) for this device: `Hip(id)` when the library sees that GPU.
pub fn hip_if_available(id: usize) -> Box<dyn Device> {
    let mut n: c_int = 0;
    let ok = unsafe { rai_hip_device_count(&mut n) } == RAI_OK && (id as c_int) < n;
    if ok && unsafe { rai_hip_init(id as c_int) } == RAI_OK {
        Box::new(Hip::new(id))
    } else {
        Box::new(Cpu)
    }
}

// ------------------------------------------------------------------------------------------------ dtypes
pub(crate) fn dtype_code(dt: &dyn DType) -> i32 {
    let any = dt.as_any();
    if any.is::<U8>() {
        RAI_U8
    } else if any.is::<U32>() {
        RAI_U32
    } else if any.is::<I64>() {
        RAI_I64
    } else if any.is::<F16>() {
        RAI_F16
    } else if any.is::<BF16>() {
        RAI_BF16
    } else if any.is::<F32>() {
        RAI_F32
    } else if any.is::<F64>() {
        RAI_F64
    } else {
        panic!("dtype {:?} has no HIP storage", dt)
    }
}

fn dtype_of(code: i32) -> &'static dyn DType {
    match code {
        RAI_U8 => &U8,
        RAI_U32 => &U32,
        RAI_I64 => &I64,
        RAI_F16 => &F16,
        RAI_BF16 => &BF16,
        RAI_F32 => &F32,
        RAI_F64 => &F64,
        _ => unreachable!("dtype code {code}"),
    }
}

fn dtype_size(code: i32) -> usize {
    match code {
        RAI_U8 => 1,
        RAI_F16 | RAI_BF16 => 2,
        RAI_U32 | RAI_F32 => 4,
        _ => 8,
    }
}

/// Element types as the C ABI takes scalars: every fill value, arange bound and exponent travels as f64.
pub trait HipScalar: Copy + 'static {
    fn to_f64_lossless(self) -> f64;
}
impl HipScalar for u8 {
    fn to_f64_lossless(self) -> f64 {
        self as f64
    }
}
impl HipScalar for u32 {
    fn to_f64_lossless(self) -> f64 {
        self as f64
    }
}
impl HipScalar for i64 {
    fn to_f64_lossless(self) -> f64 {
        self as f64 // exact up to 2^53, which covers every index and constant the models build
    }
}
impl HipScalar for f16 {
    fn to_f64_lossless(self) -> f64 {
        self.to_f64()
    }
}
impl HipScalar for bf16 {
    fn to_f64_lossless(self) -> f64 {
        self.to_f64()
    }
}
impl HipScalar for f32 {
    fn to_f64_lossless(self) -> f64 {
        self as f64
    }
}
impl HipScalar for f64 {
    fn to_f64_lossless(self) -> f64 {
        self
    }
}

// ------------------------------------------------------------------------------------------------ storage
/// A strided view of a ref-counted device allocation: what `candle_core::Tensor` is to the candle backend
/// (backend/candle.rs:18).  Views (transpose, narrow, broadcast, reshape of contiguous data) share the buffer.
pub struct HipData {
    dev: c_int,
    buf: *mut c_void, // the allocation rai_hip_alloc returned; desc.data points into it
    desc: RaiHipTensor,
    shape: Vec<usize>,
}

// The handle is only ever used from the thread that owns the (Rc-based, !Send) graph; the library itself is
// callable from any single thread.
impl HipData {
    /// Fresh contiguous storage for a node of this shape and dtype (outputs never alias inputs).
    pub fn alloc(dev: c_int, shape: &[usize], dtype: &dyn DType) -> Self {
        assert!(shape.len() <= RAI_HIP_MAX_RANK, "rank {} exceeds {}", shape.len(), RAI_HIP_MAX_RANK);
        let code = dtype_code(dtype);
        let numel: usize = shape.iter().product();
        let mut buf: *mut c_void = std::ptr::null_mut();
        check(unsafe { rai_hip_alloc(dev, (numel * dtype_size(code)).max(1), &mut buf) });
        let mut desc = RaiHipTensor { data: buf, dtype: code, rank: shape.len() as i32, shape: [1; 8], stride: [0; 8], offset: 0 };
        let mut st = 1i64;
        for i in (0..shape.len()).rev() {
            desc.shape[i] = shape[i] as i64;
            desc.stride[i] = st;
            st *= shape[i] as i64;
        }
        Self { dev, buf, desc, shape: shape.to_vec() }
    }

    /// Host bytes (already in the dtype's storage form) uploaded into fresh storage: FromArray / ToDevice<Hip>.
    pub fn from_host_bytes(dev: c_int, bytes: &[u8], shape: &[usize], dtype: &dyn DType) -> Self {
        let out = Self::alloc(dev, shape, dtype);
        assert_eq!(bytes.len(), out.numel() * dtype_size(out.desc.dtype), "byte count does not match the shape");
        if !bytes.is_empty() {
            check(unsafe { rai_hip_h2d(dev, out.buf, bytes.as_ptr() as *const c_void, bytes.len()) });
        }
        out
    }

    /// Storage that the library's graph evaluator produced (backend/hip_graph.rs): `desc` is a view into `buf`, an
    /// allocation of rai_hip_alloc, which this handle retains.
    pub(crate) fn adopt(dev: c_int, buf: *mut c_void, desc: RaiHipTensor) -> Self {
        check(unsafe { rai_hip_retain(buf) });
        let shape = desc.shape[..desc.rank as usize].iter().map(|&d| d as usize).collect();
        Self { dev, buf, desc, shape }
    }

    /// The allocation the view points into.
    pub(crate) fn buffer(&self) -> *mut c_void {
        self.buf
    }

    /// Another view of the same allocation.
    fn view(&self, desc: RaiHipTensor) -> Self {
        check(unsafe { rai_hip_retain(self.buf) });
        let shape = desc.shape[..desc.rank as usize].iter().map(|&d| d as usize).collect();
        Self { dev: self.dev, buf: self.buf, desc, shape }
    }

    pub fn desc(&self) -> &RaiHipTensor {
        &self.desc
    }

    pub fn numel(&self) -> usize {
        self.shape.iter().product()
    }

    pub fn is_contiguous(&self) -> bool {
        let mut expect = 1i64;
        for i in (0..self.shape.len()).rev() {
            if self.desc.shape[i] == 1 {
                continue;
            }
            if self.desc.stride[i] != expect {
                return false;
            }
            expect *= self.desc.shape[i];
        }
        true
    }

    /// A contiguous copy (or another handle to `self` when it already is contiguous).
    pub fn contiguous(&self) -> Self {
        if self.is_contiguous() {
            return self.view(self.desc);
        }
        let out = Self::alloc(self.dev, &self.shape, dtype_of(self.desc.dtype));
        check(unsafe { rai_hip_copy(self.dev, &self.desc, &out.desc) });
        out
    }

    // ---- zero-copy views: what candle layouts give the reference backend (candle.rs:555-593, 891-899)
    fn transpose(&self, d0: usize, d1: usize) -> Self {
        let mut d = self.desc;
        d.shape.swap(d0, d1);
        d.stride.swap(d0, d1);
        self.view(d)
    }

    fn permute(&self, dims: &[usize]) -> Self {
        let mut d = self.desc;
        for (i, &p) in dims.iter().enumerate() {
            d.shape[i] = self.desc.shape[p];
            d.stride[i] = self.desc.stride[p];
        }
        self.view(d)
    }

    fn narrow(&self, dim: usize, start: usize, len: usize) -> Self {
        assert!(start + len <= self.shape[dim], "narrow out of range");
        let mut d = self.desc;
        d.shape[dim] = len as i64;
        d.offset += start as i64 * d.stride[dim];
        self.view(d)
    }

    fn broadcast_as(&self, shape: &[usize]) -> Self {
        let pad = shape.len() - self.shape.len();
        let mut d = self.desc;
        d.rank = shape.len() as i32;
        for i in 0..shape.len() {
            let (s, st) = if i < pad { (1, 0) } else { (self.desc.shape[i - pad], self.desc.stride[i - pad]) };
            d.shape[i] = shape[i] as i64;
            d.stride[i] = if s == shape[i] as i64 { st } else { assert_eq!(s, 1, "cannot broadcast"); 0 };
        }
        self.view(d)
    }

    /// Reshape: a view when the data is contiguous, else of a contiguous copy (candle.rs:565-573).
    fn reshape(&self, shape: &[usize]) -> Self {
        let src = self.contiguous();
        let mut d = src.desc;
        d.rank = shape.len() as i32;
        d.shape = [1; 8];
        d.stride = [0; 8];
        let mut st = 1i64;
        for i in (0..shape.len()).rev() {
            d.shape[i] = shape[i] as i64;
            d.stride[i] = st;
            st *= shape[i] as i64;
        }
        src.view(d)
    }

    /// Device -> host: a synchronous copy of the contiguous contents (as_bytes / as_vec / as_scalar).
    fn host_bytes(&self) -> Vec<u8> {
        let src = self.contiguous();
        let es = dtype_size(src.desc.dtype);
        let mut out = vec![0u8; src.numel() * es];
        if !out.is_empty() {
            let base = unsafe { (src.desc.data as *const u8).add(src.desc.offset as usize * es) };
            check(unsafe { rai_hip_d2h(src.dev, out.as_mut_ptr() as *mut c_void, base as *const c_void, out.len()) });
        }
        out
    }

    fn host_vec<T: Copy>(&self) -> Vec<T> {
        let bytes = self.host_bytes();
        let n = bytes.len() / std::mem::size_of::<T>();
        let mut v = Vec::<T>::with_capacity(n);
        unsafe {
            std::ptr::copy_nonoverlapping(bytes.as_ptr(), v.as_mut_ptr() as *mut u8, bytes.len());
            v.set_len(n);
        }
        v
    }
}

impl Clone for HipData {
    fn clone(&self) -> Self {
        self.view(self.desc)
    }
}

impl Drop for HipData {
    fn drop(&mut self) {
        // stream-ordered: the block returns to the pool and later work on the stream runs after its readers
        unsafe { rai_hip_release(self.buf) };
    }
}

impl Debug for HipData {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipData(dev={}, dtype={:?}, shape={:?})", self.dev, dtype_of(self.desc.dtype), self.shape)
    }
}

impl Display for HipData {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        match self.desc.dtype {
            RAI_U8 => write!(f, "{:?}", self.host_vec::<u8>()),
            RAI_U32 => write!(f, "{:?}", self.host_vec::<u32>()),
            RAI_I64 => write!(f, "{:?}", self.host_vec::<i64>()),
            RAI_F16 => write!(f, "{:?}", self.host_vec::<f16>()),
            RAI_BF16 => write!(f, "{:?}", self.host_vec::<bf16>()),
            RAI_F32 => write!(f, "{:?}", self.host_vec::<f32>()),
            _ => write!(f, "{:?}", self.host_vec::<f64>()),
        }
    }
}

impl TensorLike for HipData {
    fn as_any(&self) -> &dyn Any {
        self
    }

    fn shape(&self) -> &[usize] {
        &self.shape
    }

    fn dtype(&self) -> &dyn DType {
        dtype_of(self.desc.dtype)
    }

    fn as_scalar(&self) -> Box<dyn Any> {
        match self.desc.dtype {
            RAI_U8 => Box::new(self.host_vec::<u8>()[0]),
            RAI_U32 => Box::new(self.host_vec::<u32>()[0]),
            RAI_I64 => Box::new(self.host_vec::<i64>()[0]),
            RAI_F16 => Box::new(self.host_vec::<f16>()[0]),
            RAI_BF16 => Box::new(self.host_vec::<bf16>()[0]),
            RAI_F32 => Box::new(self.host_vec::<f32>()[0]),
            _ => Box::new(self.host_vec::<f64>()[0]),
        }
    }

    fn as_vec(&self) -> Box<dyn Any> {
        match self.desc.dtype {
            RAI_U8 => Box::new(self.host_vec::<u8>()),
            RAI_U32 => Box::new(self.host_vec::<u32>()),
            RAI_I64 => Box::new(self.host_vec::<i64>()),
            RAI_F16 => Box::new(self.host_vec::<f16>()),
            RAI_BF16 => Box::new(self.host_vec::<bf16>()),
            RAI_F32 => Box::new(self.host_vec::<f32>()),
            _ => Box::new(self.host_vec::<f64>()),
        }
    }

    fn as_bytes(&self) -> Vec<u8> {
        self.host_bytes()
    }
}

// ------------------------------------------------------------------------------------------------ backend
#[derive(Debug, Clone, Copy, Default, PartialEq, Eq)]
pub struct HipBackend;

impl Backend for HipBackend {
    fn clone_boxed(&self) -> Box<dyn Backend> {
        Box::new(*self)
    }

    fn as_any(&self) -> &dyn Any {
        self
    }

    #[inline]
    fn data_type_id(&self) -> TypeId {
        TypeId::of::<HipData>()
    }

    fn equal(&self, rhs: &dyn Backend) -> bool {
        rhs.as_any().downcast_ref().map_or(false, |other| self == other)
    }
}

#[inline]
fn data(t: &Tensor) -> impl Deref<Target = HipData> + '_ {
    t.get_data::<HipData>().expect("input of a Hip primitive is evaluated and lives on a Hip device")
}

#[inline]
fn fresh(dev: &Hip, output: &Tensor) -> HipData {
    HipData::alloc(dev.dev(), output.shape(), output.dtype())
}

// ---- creation (candle.rs:197-273)
impl<T: Type> Eval<Hip, ops::Full<T>> for HipBackend
where
    T::Repr: HipScalar,
{
    fn eval(&self, dev: &Hip, op: &ops::Full<T>, _: &[Tensor], output: &Tensor) {
        let out = fresh(dev, output);
        check(unsafe { rai_hip_fill(dev.dev(), out.desc(), op.val.to_f64_lossless()) });
        output.set_data(out);
    }
}

impl<T: Type> Eval<Hip, ops::Arange<T>> for HipBackend
where
    T::Repr: HipScalar,
{
    fn eval(&self, dev: &Hip, op: &ops::Arange<T>, _: &[Tensor], output: &Tensor) {
        let out = fresh(dev, output); // the length was fixed by ops/arange.rs:102-117
        check(unsafe { rai_hip_arange(dev.dev(), out.desc(), op.start.to_f64_lossless(), op.step.to_f64_lossless()) });
        output.set_data(out);
    }
}

impl<T: Type> Eval<Hip, ops::FromArray<T>> for HipBackend
where
    T::Repr: HipScalar,
{
    fn eval(&self, dev: &Hip, op: &ops::FromArray<T>, _: &[Tensor], output: &Tensor) {
        let bytes = unsafe {
            std::slice::from_raw_parts(op.data.as_ptr() as *const u8, op.data.len() * std::mem::size_of::<T::Repr>())
        };
        output.set_data(HipData::from_host_bytes(dev.dev(), bytes, output.shape(), output.dtype()));
    }
}

// ---- ToDevice (candle.rs:776-790).  The node lives on the TARGET device (ops/to_device.rs:48-59), so
// `ToDevice<Hip>` is looked up under `Hip`; its input may live on the host (any TensorLike: as_bytes is the
// storage form the upload wants), on the same GPU or on another one.
impl Eval<Hip, ops::ToDevice<Hip>> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::ToDevice<Hip>, inputs: &[Tensor], output: &Tensor) {
        let x = &inputs[0];
        let dst = op.device.dev();
        if let Some(src_hip) = x.device().as_any().downcast_ref::<Hip>() {
            let src = data(x);
            let out = HipData::alloc(dst, output.shape(), output.dtype());
            check(unsafe { rai_hip_to_device(src_hip.dev(), src.desc(), dst, out.desc()) });
            output.set_data(out);
        } else {
            // any other backend's storage: its bytes in the dtype's storage form (tensor.rs:352-370, the same
            // accessor Module::to_safetensors uses)
            let bytes = safetensors::View::data(&x);
            output.set_data(HipData::from_host_bytes(dst, &bytes, output.shape(), output.dtype()));
        }
    }
}

/// `ToDevice<Cpu>` of a tensor that lives on `Hip`: registered under `Cpu` IN PLACE of the candle rule for that
/// pair, it downloads Hip data and hands everything else to the candle backend unchanged.
#[derive(Debug, Clone, Copy, Default, PartialEq, Eq)]
pub struct HipToCpu;

impl Eval<Cpu, ops::ToDevice<Cpu>> for HipToCpu {
    fn eval(&self, dev: &Cpu, op: &ops::ToDevice<Cpu>, inputs: &[Tensor], output: &Tensor) {
        let x = &inputs[0];
        if x.device().as_any().is::<Hip>() {
            // the host image becomes an ordinary FromArray tensor on Cpu (evaluated by the candle rule) whose data
            // is then moved into the output node (tensor.rs:126-148)
            let d = data(x);
            let shape = output.shape().to_vec();
            let host = match d.desc.dtype {
                RAI_U8 => Tensor::from_array(d.host_vec::<u8>(), shape, dev),
                RAI_U32 => Tensor::from_array(d.host_vec::<u32>(), shape, dev),
                RAI_I64 => Tensor::from_array(d.host_vec::<i64>(), shape, dev),
                RAI_F16 => Tensor::from_array(d.host_vec::<f16>(), shape, dev),
                RAI_BF16 => Tensor::from_array(d.host_vec::<bf16>(), shape, dev),
                RAI_F32 => Tensor::from_array(d.host_vec::<f32>(), shape, dev),
                _ => Tensor::from_array(d.host_vec::<f64>(), shape, dev),
            };
            drop(d);
            output.replace_data(host).expect("download from Hip");
        } else {
            <CandleBackend as Eval<Cpu, ops::ToDevice<Cpu>>>::eval(&CandleBackend, dev, op, inputs, output);
        }
    }
}

// ---- elementwise binary (candle.rs:275-325, 658-760): operands arrive already broadcast to the output shape
macro_rules! hip_binary {
    ($($op:ident => $code:ident),* $(,)?) => {$(
        impl Eval<Hip, ops::$op> for HipBackend {
            fn eval(&self, dev: &Hip, _: &ops::$op, inputs: &[Tensor], output: &Tensor) {
                let (a, b) = (data(&inputs[0]), data(&inputs[1]));
                let out = fresh(dev, output);
                check(unsafe { rai_hip_binary(dev.dev(), $code, a.desc(), b.desc(), out.desc()) });
                output.set_data(out);
            }
        }
    )*};
}
hip_binary!(Add => RAI_BIN_ADD, Sub => RAI_BIN_SUB, Mul => RAI_BIN_MUL, Div => RAI_BIN_DIV,
            Maximum => RAI_BIN_MAXIMUM, Minimum => RAI_BIN_MINIMUM,
            Equal => RAI_BIN_EQ, NotEqual => RAI_BIN_NE, Greater => RAI_BIN_GT, GreaterEqual => RAI_BIN_GE,
            Less => RAI_BIN_LT, LessEqual => RAI_BIN_LE);

// ---- elementwise unary (candle.rs:445-473, 525-553, 595-656, 947-964)
macro_rules! hip_unary {
    ($($op:ident => $code:ident),* $(,)?) => {$(
        impl Eval<Hip, ops::$op> for HipBackend {
            fn eval(&self, dev: &Hip, _: &ops::$op, inputs: &[Tensor], output: &Tensor) {
                let x = data(&inputs[0]);
                let out = fresh(dev, output);
                check(unsafe { rai_hip_unary(dev.dev(), $code, x.desc(), out.desc(), 0.0) });
                output.set_data(out);
            }
        }
    )*};
}
hip_unary!(Sin => RAI_UN_SIN, Cos => RAI_UN_COS, Tanh => RAI_UN_TANH, Negative => RAI_UN_NEG, Square => RAI_UN_SQUARE,
           Sqrt => RAI_UN_SQRT, Rsqrt => RAI_UN_RSQRT, Sign => RAI_UN_SIGN, Abs => RAI_UN_ABS, Exp => RAI_UN_EXP,
           Log => RAI_UN_LOG, Log2 => RAI_UN_LOG2, Log10 => RAI_UN_LOG10, Erf => RAI_UN_ERF);

impl<T: Type> Eval<Hip, ops::Powf<T>> for HipBackend
where
    T::Repr: FloatElemType,
{
    fn eval(&self, dev: &Hip, op: &ops::Powf<T>, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output);
        check(unsafe { rai_hip_unary(dev.dev(), RAI_UN_POWF, x.desc(), out.desc(), op.exponent.to_f64()) });
        output.set_data(out);
    }
}

impl<T: Type> Eval<Hip, ops::ToDType<T>> for HipBackend {
    fn eval(&self, dev: &Hip, _: &ops::ToDType<T>, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output);
        check(unsafe { rai_hip_cast(dev.dev(), x.desc(), out.desc()) });
        output.set_data(out);
    }
}

// ---- contraction (candle.rs:327-443).  The kernel takes any strides for the last two dims and stride-0 batch
// dims, so nothing is made contiguous first and no input is overwritten.
impl Eval<Hip, ops::MatMul> for HipBackend {
    fn eval(&self, dev: &Hip, _: &ops::MatMul, inputs: &[Tensor], output: &Tensor) {
        let (a, b) = (data(&inputs[0]), data(&inputs[1]));
        let out = fresh(dev, output);
        // leading dims were broadcast by ops/matmul.rs:34-70 (shape.rs:130-160); present both operands at the
        // output's rank
        let lead = &output.shape()[..output.shape().len() - 2];
        let (a2, b2) = (batch_view(&a, lead), batch_view(&b, lead));
        check(unsafe { rai_hip_matmul(dev.dev(), a2.desc(), b2.desc(), out.desc()) });
        output.set_data(out);
    }
}

fn batch_view(x: &HipData, lead: &[usize]) -> HipData {
    let r = x.shape.len();
    let mut full = lead.to_vec();
    full.extend_from_slice(&x.shape[r - 2..]);
    if full == x.shape {
        x.clone()
    } else {
        x.broadcast_as(&full)
    }
}

// ---- reductions (candle.rs:475-523, 793-836, 917-944)
fn reduce(dev: &Hip, code: i32, dims: &[usize], keep_dim: bool, inputs: &[Tensor], output: &Tensor) {
    let x = data(&inputs[0]);
    let out = fresh(dev, output);
    let d: Vec<i32> = dims.iter().map(|&d| d as i32).collect();
    check(unsafe { rai_hip_reduce(dev.dev(), code, x.desc(), d.as_ptr(), d.len() as i32, keep_dim as i32, out.desc()) });
    output.set_data(out);
}

impl Eval<Hip, ops::ReduceSum> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ReduceSum, inputs: &[Tensor], output: &Tensor) {
        reduce(dev, RAI_RED_SUM, op.dims(), op.keep_dim, inputs, output);
    }
}
impl Eval<Hip, ops::ReduceMax> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ReduceMax, inputs: &[Tensor], output: &Tensor) {
        reduce(dev, RAI_RED_MAX, op.dims(), op.keep_dim, inputs, output);
    }
}
impl Eval<Hip, ops::ReduceMin> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ReduceMin, inputs: &[Tensor], output: &Tensor) {
        reduce(dev, RAI_RED_MIN, op.dims(), op.keep_dim, inputs, output);
    }
}

impl Eval<Hip, ops::Softmax> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::Softmax, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output);
        check(unsafe { rai_hip_softmax(dev.dev(), x.desc(), op.dim as i32, out.desc()) });
        output.set_data(out);
    }
}
impl Eval<Hip, ops::LogSoftmax> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::LogSoftmax, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output);
        check(unsafe { rai_hip_log_softmax(dev.dev(), x.desc(), op.dim as i32, out.desc()) });
        output.set_data(out);
    }
}

impl Eval<Hip, ops::ArgMax> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ArgMax, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output); // U32, ops/argmax.rs:48-61
        check(unsafe { rai_hip_argmax(dev.dev(), x.desc(), op.dim() as i32, op.keep_dim as i32, out.desc()) });
        output.set_data(out);
    }
}
impl Eval<Hip, ops::ArgMin> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ArgMin, inputs: &[Tensor], output: &Tensor) {
        let x = data(&inputs[0]);
        let out = fresh(dev, output);
        // the reference's candle rule calls argmax here (candle.rs:932-944, an upstream slip); this one is argmin
        check(unsafe { rai_hip_argmin(dev.dev(), x.desc(), op.dim() as i32, op.keep_dim as i32, out.desc()) });
        output.set_data(out);
    }
}

// ---- indexing (candle.rs:838-915, 990-1004)
impl Eval<Hip, ops::IndexSelect> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::IndexSelect, inputs: &[Tensor], output: &Tensor) {
        let (x, index) = (data(&inputs[0]), data(&inputs[1]));
        let out = fresh(dev, output);
        check(unsafe { rai_hip_index_select(dev.dev(), x.desc(), index.desc(), op.dim as i32, out.desc()) });
        // an index outside the table is reported by the library, never read silently
        let mut bad = 0u64;
        check(unsafe { rai_hip_index_errors(dev.dev(), &mut bad) });
        assert!(bad == 0, "index_select: {bad} indices out of range");
        output.set_data(out);
    }
}

impl Eval<Hip, ops::Gather> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::Gather, inputs: &[Tensor], output: &Tensor) {
        let (x, index) = (data(&inputs[0]).contiguous(), data(&inputs[1]).contiguous());
        let out = fresh(dev, output);
        check(unsafe { rai_hip_gather(dev.dev(), x.desc(), index.desc(), op.dim as i32, out.desc()) });
        output.set_data(out);
    }
}

impl Eval<Hip, ops::IndexAdd> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::IndexAdd, inputs: &[Tensor], output: &Tensor) {
        // inputs are ordered [x, source, index] (ops/index_add.rs:57-59)
        let (x, source, index) =
            (data(&inputs[0]).contiguous(), data(&inputs[1]).contiguous(), data(&inputs[2]).contiguous());
        let out = fresh(dev, output);
        check(unsafe { rai_hip_index_add(dev.dev(), x.desc(), index.desc(), source.desc(), op.dim as i32, out.desc()) });
        output.set_data(out);
    }
}

impl Eval<Hip, ops::ScatterAdd> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::ScatterAdd, inputs: &[Tensor], output: &Tensor) {
        // inputs are ordered [x, updates, indices] (ops/scatter_add.rs:57)
        let (x, source, index) =
            (data(&inputs[0]).contiguous(), data(&inputs[1]).contiguous(), data(&inputs[2]).contiguous());
        let out = fresh(dev, output);
        check(unsafe { rai_hip_scatter_add(dev.dev(), x.desc(), index.desc(), source.desc(), op.dim as i32, out.desc()) });
        output.set_data(out);
    }
}

impl Eval<Hip, ops::Where> for HipBackend {
    fn eval(&self, dev: &Hip, _: &ops::Where, inputs: &[Tensor], output: &Tensor) {
        // inputs are ordered [on_true, on_false, cond] (ops/where.rs:37-45)
        let (on_true, on_false, cond) = (data(&inputs[0]), data(&inputs[1]), data(&inputs[2]));
        let out = fresh(dev, output);
        check(unsafe { rai_hip_where(dev.dev(), cond.desc(), on_true.desc(), on_false.desc(), out.desc()) });
        output.set_data(out);
    }
}

impl Eval<Hip, ops::Concatenate> for HipBackend {
    fn eval(&self, dev: &Hip, op: &ops::Concatenate, inputs: &[Tensor], output: &Tensor) {
        // one strided copy per piece into the slice of the output it fills (candle.rs:880-889)
        let out = fresh(dev, output);
        let mut at = 0usize;
        for t in inputs {
            let x = data(t);
            let len = x.shape[op.dim];
            let dst = out.narrow(op.dim, at, len);
            check(unsafe { rai_hip_copy(dev.dev(), x.desc(), dst.desc()) });
            at += len;
        }
        output.set_data(out);
    }
}

// ---- views: metadata only, like candle's layouts (candle.rs:555-593, 891-899, 980-988)
impl Eval<Hip, ops::Transpose> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::Transpose, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).transpose(op.dim0, op.dim1));
    }
}
impl Eval<Hip, ops::Permute> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::Permute, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).permute(op.dims()));
    }
}
impl Eval<Hip, ops::Narrow> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::Narrow, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).narrow(op.dim, op.start, op.len));
    }
}
impl Eval<Hip, ops::Broadcast> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::Broadcast, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).broadcast_as(op.shape()));
    }
}
impl Eval<Hip, ops::Reshape> for HipBackend {
    fn eval(&self, _: &Hip, op: &ops::Reshape, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).reshape(op.shape()));
    }
}
impl Eval<Hip, ops::ToContiguous> for HipBackend {
    fn eval(&self, _: &Hip, _: &ops::ToContiguous, inputs: &[Tensor], output: &Tensor) {
        output.set_data(data(&inputs[0]).contiguous());
    }
}

// ------------------------------------------------------------------------------------------------ registration
/// The `Hip` rows of `EVAL_DISPATCHER` (dispatch.rs:159-179): the op list of `register_backend!`
/// (dispatch.rs:41-157) minus `Random<_>`, `Normal<_>`, `Conv1d`, `Conv2d`, `ConvTranspose1d`, `ConvTranspose2d`,
/// `MaxPool1d`, `MaxPool2d`, `AvgPool1d`, `AvgPool2d`, `UpsampleNearest1d`, `UpsampleNearest2d` and
/// `FlashAttention`, for which there is no HIP kernel: evaluating one of
/// those on `Hip` reports `Error::Unimplemented` (eval.rs:40-43).  (`Normal<BF16>` is not registered for any
/// device in the reference either, dispatch.rs:55-57: bf16 models load or cast their weights.)
pub(crate) fn register_hip(rules: &mut HashMap<(TypeId, TypeId), DynBackend>) {
    use crate::dispatch::_register as reg;
    let b = HipBackend;
    macro_rules! per_dtype {
        ($op:ident: $($t:ident),*) => {$( reg::<HipBackend, Hip, ops::$op<$t>>(b, rules); )*};
    }
    macro_rules! plain {
        ($($op:ident),* $(,)?) => {$( reg::<HipBackend, Hip, ops::$op>(b, rules); )*};
    }
    // creation
    per_dtype!(Full: U8, U32, BF16, F16, F32, F64, I64);
    per_dtype!(Arange: U8, U32, BF16, F16, F32, F64, I64);
    per_dtype!(FromArray: U8, U32, BF16, F16, F32, F64, I64);
    plain!(Concatenate);
    // binary
    plain!(Add, Sub, Mul, Div, MatMul, Equal, NotEqual, Greater, GreaterEqual, Less, LessEqual, Maximum, Minimum);
    // unary
    plain!(Sin, Cos, Tanh, Negative, Square, Sqrt, Rsqrt, Sign, Abs, Exp, Log, Log2, Log10, Erf, Softmax, LogSoftmax);
    per_dtype!(Powf: BF16, F16, F32, F64);
    per_dtype!(ToDType: U8, U32, BF16, F16, F32, F64, I64);
    // device transfers: into Hip from anywhere, and out of Hip to the host
    reg::<HipBackend, Hip, ops::ToDevice<Hip>>(b, rules);
    reg::<HipToCpu, Cpu, ops::ToDevice<Cpu>>(HipToCpu, rules);
    // indexing
    plain!(Gather, IndexSelect, Narrow, Where, ScatterAdd, IndexAdd);
    // transform
    plain!(Transpose, Reshape, Permute, Broadcast, ToContiguous);
    // reduce
    plain!(ReduceSum, ReduceMax, ReduceMin, ArgMax, ArgMin);
}
