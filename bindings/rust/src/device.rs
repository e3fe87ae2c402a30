//! The device: one slhip context (one in-order HIP stream) plus the custos modules it is
//! composed with.  Mirrors how the reference composes `OpenCL<Mods>` / `CPU<Mods>`
//! (`examples/sine_net.rs:124`: `CPU::<Autograd<Cached<Base>>>::new()`).
use core::ffi::c_void;
use custos::{
    flag::AllocFlag, Alloc, Base, Buffer, ClearBuf, CloneBuf, Device, HasId, Id, Module, OnDropBuffer, PtrType, Read,
    Setup, ShallowCopy, Shape, WriteBuf,
};

use crate::{check, ffi};

#[derive(Debug, Clone)]
pub struct HipError {
    pub status: i32,
    pub msg: String,
}
impl std::fmt::Display for HipError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "sliced_hip status {}: {}", self.status, self.msg)
    }
}
impl std::error::Error for HipError {}

/// A device allocation of `len` elements.  `flag` follows custos: only `AllocFlag::None`
/// allocations are freed on drop (wrappers and cache-owned views are not).
pub struct HipPtr<T> {
    pub ptr: *mut T,
    pub len: usize,
    pub flag: AllocFlag,
    pub ctx: *mut ffi::SlhipCtx,
}

impl<T> Default for HipPtr<T> {
    fn default() -> Self {
        HipPtr { ptr: core::ptr::null_mut(), len: 0, flag: AllocFlag::default(), ctx: core::ptr::null_mut() }
    }
}
impl<T> PtrType for HipPtr<T> {
    fn size(&self) -> usize {
        self.len
    }
    fn flag(&self) -> AllocFlag {
        self.flag
    }
}
impl<T> HasId for HipPtr<T> {
    fn id(&self) -> Id {
        // custos: an Id is the allocation's address plus its length
        Id { id: self.ptr as u64, len: self.len }
    }
}
impl<T> ShallowCopy for HipPtr<T> {
    unsafe fn shallow(&self) -> Self {
        HipPtr { ptr: self.ptr, len: self.len, flag: AllocFlag::Wrapper, ctx: self.ctx }
    }
}
impl<T> Drop for HipPtr<T> {
    fn drop(&mut self) {
        if self.flag != AllocFlag::None || self.ptr.is_null() {
            return;
        }
        // slhip_free waits for the stream, so work that still reads the buffer finishes first
        unsafe { ffi::slhip_free(self.ctx, self.ptr as *mut c_void) };
    }
}

/// The device.  `modules` is the custos module stack (`Base`, `Cached<..>`, `Autograd<..>`).
pub struct HIP<Mods = Base> {
    pub modules: Mods,
    pub ctx: *mut ffi::SlhipCtx,
}

impl<SimpleMods> HIP<SimpleMods> {
    /// `HIP::<Autograd<Cached<Base>>>::new(0)`: device `ordinal` must be a gfx950 GPU.
    pub fn new<NewMods>(ordinal: i32) -> Result<HIP<NewMods>, HipError>
    where
        SimpleMods: Module<HIP, Module = NewMods>,
        NewMods: Setup<HIP<NewMods>>,
    {
        let mut ctx = core::ptr::null_mut();
        check(unsafe { ffi::slhip_init(ordinal, &mut ctx) })?;
        let mut dev = HIP { modules: SimpleMods::new(), ctx };
        NewMods::setup(&mut dev).map_err(|e| HipError { status: ffi::SLHIP_EINVAL, msg: e.to_string() })?;
        Ok(dev)
    }
}

impl<Mods> HIP<Mods> {
    /// Waits for everything issued on this device.
    pub fn sync(&self) -> Result<(), HipError> {
        check(unsafe { ffi::slhip_sync(self.ctx) })
    }
    pub fn name(&self) -> String {
        let mut buf = [0 as std::os::raw::c_char; 128];
        unsafe { ffi::slhip_device_name(self.ctx, buf.as_mut_ptr(), buf.len()) };
        unsafe { std::ffi::CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }
    /// Seeded uniform fill on the device (replaces `RandOp::rand`, src/rawops/cpu/rand.rs:7-12,
    /// whose generator is unseeded).
    pub fn rand_uniform<S: Shape>(&self, x: &mut Buffer<f32, Self, S>, seed: u64, tag: u64, lo: f32, hi: f32) {
        check(unsafe { ffi::slhip_rand_uniform(self.ctx, seed, tag, lo, hi, x.len(), x.ptr_mut()) }).unwrap();
    }
    /// `SGD::step` of the examples on the device (examples/sine_net.rs:105-116): `p -= g * lr`
    /// for a whole parameter list in one launch per eight tensors.
    pub fn sgd_step<S: Shape>(&self, params: &mut [&mut Buffer<f32, Self, S>], lr: f32)
    where
        Self: Device,
    {
        let ps: Vec<*mut f32> = params.iter_mut().map(|p| p.ptr_mut()).collect();
        let gs: Vec<*const f32> = params.iter().map(|p| p.grad().ptr()).collect();
        let ns: Vec<usize> = params.iter().map(|p| p.len()).collect();
        check(unsafe { ffi::slhip_sgd_step_multi(self.ctx, ps.len(), ps.as_ptr(), gs.as_ptr(), ns.as_ptr(), lr) }).unwrap();
    }
}

impl<Mods> HIP<Mods> {
    /// One whole training step of the sine-fit loop (examples/sine_net.rs:119-166) as two launches:
    /// forward through three Linear layers with ReLU between them, the MSE loss into `loss[0]`,
    /// backward and SGD on the six parameter buffers in place; their gradient buffers receive the
    /// step's gradients.  Layers of more than 64 hidden units or 8 inputs / outputs come back as
    /// `Err` (status `SLHIP_EINVAL`): run the op traits one by one then.
    #[allow(clippy::too_many_arguments)]
    pub fn mlp3_mse_step<S: Shape>(
        &self,
        batch: usize,
        d_in: usize,
        d_h: usize,
        d_out: usize,
        x: &Buffer<f32, Self, S>,
        target: &Buffer<f32, Self, S>,
        params: &mut [&mut Buffer<f32, Self, S>; 6],
        lr: f32,
        loss: &mut Buffer<f32, Self, S>,
    ) -> Result<(), HipError>
    where
        Self: Device,
    {
        let grads: Vec<*mut f32> = params.iter_mut().map(|p| p.grad_mut().ptr_mut()).collect();
        let p: Vec<*mut f32> = params.iter_mut().map(|p| p.ptr_mut()).collect();
        check(unsafe {
            ffi::slhip_mlp3_mse_step(self.ctx, batch, d_in, d_h, d_out, x.ptr(), target.ptr(), p[0], p[1], p[2], p[3], p[4], p[5],
                                     grads.as_ptr(), lr, loss.ptr_mut())
        })
    }
    /// Which kernel and plan the last product on this device ran as (for logs).
    pub fn last_gemm_plan(&self) -> String {
        let mut buf = [0 as std::os::raw::c_char; 256];
        unsafe { ffi::slhip_gemm_plan_describe(self.ctx, buf.as_mut_ptr(), buf.len()) };
        unsafe { std::ffi::CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }
}

impl<Mods> Drop for HIP<Mods> {
    fn drop(&mut self) {
        unsafe { ffi::slhip_destroy(self.ctx) };
    }
}

impl<Mods: OnDropBuffer> Device for HIP<Mods> {
    type Base<T, S: Shape> = HipPtr<T>;
    type Data<T, S: Shape> = Self::Base<T, S>;
    type Error = HipError;

    fn new() -> Result<Self, Self::Error> {
        // custos: devices are built through `HIP::<Mods>::new(ordinal)` above
        Err(HipError { status: ffi::SLHIP_EINVAL, msg: "use HIP::<Mods>::new(ordinal)".into() })
    }
    #[inline(always)]
    fn base_to_data<T, S: Shape>(&self, base: Self::Base<T, S>) -> Self::Data<T, S> {
        base
    }
    #[inline(always)]
    fn wrap_to_data<T, S: Shape>(&self, wrap: Self::Base<T, S>) -> Self::Data<T, S> {
        wrap
    }
    #[inline(always)]
    fn data_as_wrap<T, S: Shape>(data: &Self::Data<T, S>) -> &Self::Base<T, S> {
        data
    }
    #[inline(always)]
    fn data_as_wrap_mut<T, S: Shape>(data: &mut Self::Data<T, S>) -> &mut Self::Base<T, S> {
        data
    }
}

impl<Mods: OnDropBuffer, T> Alloc<T> for HIP<Mods> {
    /// `retrieve` hands out zeroed memory on the reference's CPU device, and `slice_sum_rows2`
    /// accumulates into it (src/ops2/sum/cpu.rs:78-84): new allocations are zeroed here too.
    fn alloc<S: Shape>(&self, len: usize, flag: AllocFlag) -> Self::Base<T, S> {
        assert!(len > 0, "invalid buffer len: 0");
        let bytes = len * core::mem::size_of::<T>();
        let mut p: *mut c_void = core::ptr::null_mut();
        check(unsafe { ffi::slhip_malloc(self.ctx, bytes, &mut p) }).unwrap();
        check(unsafe { ffi::slhip_memset(self.ctx, p, 0, bytes) }).unwrap();
        HipPtr { ptr: p as *mut T, len, flag, ctx: self.ctx }
    }
    fn alloc_from_slice<S: Shape>(&self, data: &[T]) -> Self::Base<T, S>
    where
        T: Clone,
    {
        let bytes = core::mem::size_of_val(data);
        let mut p: *mut c_void = core::ptr::null_mut();
        check(unsafe { ffi::slhip_malloc(self.ctx, bytes, &mut p) }).unwrap();
        check(unsafe { ffi::slhip_memcpy_h2d(self.ctx, p, data.as_ptr() as *const c_void, bytes) }).unwrap();
        HipPtr { ptr: p as *mut T, len: data.len(), flag: AllocFlag::None, ctx: self.ctx }
    }
}

impl<Mods: OnDropBuffer, T: Clone + Default, S: Shape> Read<T, S> for HIP<Mods> {
    type Read<'a> = Vec<T> where T: 'a, S: 'a, Self: 'a;
    fn read<'a>(&self, buf: &'a Buffer<T, Self, S>) -> Self::Read<'a> {
        self.read_to_vec(buf)
    }
    fn read_to_vec(&self, buf: &Buffer<T, Self, S>) -> Vec<T> {
        let mut v = vec![T::default(); buf.len()];
        let bytes = buf.len() * core::mem::size_of::<T>();
        // waits for the stream: everything issued before is visible in the copy
        check(unsafe { ffi::slhip_memcpy_d2h(self.ctx, v.as_mut_ptr() as *mut c_void, buf.ptr() as *const c_void, bytes) })
            .unwrap();
        v
    }
}

impl<Mods: OnDropBuffer, T, S: Shape> WriteBuf<T, S> for HIP<Mods> {
    fn write(&self, buf: &mut Buffer<T, Self, S>, data: &[T]) {
        assert_eq!(buf.len(), data.len());
        let bytes = core::mem::size_of_val(data);
        check(unsafe { ffi::slhip_memcpy_h2d(self.ctx, buf.ptr_mut() as *mut c_void, data.as_ptr() as *const c_void, bytes) })
            .unwrap();
    }
    fn write_buf(&self, dst: &mut Buffer<T, Self, S>, src: &Buffer<T, Self, S>) {
        assert_eq!(dst.len(), src.len());
        let bytes = dst.len() * core::mem::size_of::<T>();
        check(unsafe { ffi::slhip_memcpy_d2d(self.ctx, dst.ptr_mut() as *mut c_void, src.ptr() as *const c_void, bytes) })
            .unwrap();
    }
}

impl<Mods: OnDropBuffer, T, S: Shape> ClearBuf<T, S> for HIP<Mods> {
    fn clear(&self, buf: &mut Buffer<T, Self, S>) {
        let bytes = buf.len() * core::mem::size_of::<T>();
        check(unsafe { ffi::slhip_memset(self.ctx, buf.ptr_mut() as *mut c_void, 0, bytes) }).unwrap();
    }
}

impl<'a, Mods: OnDropBuffer + 'a, T: 'a, S: Shape + 'a> CloneBuf<'a, T, S> for HIP<Mods> {
    fn clone_buf(&'a self, buf: &Buffer<'a, T, Self, S>) -> Buffer<'a, T, Self, S> {
        let mut out = Buffer::new(self, buf.len());
        self.write_buf(&mut out, buf);
        out
    }
}

// custos: the pass-through impls (Retrieve/Retriever, AddOperation, AddGradFn, MayTapeActions,
// ZeroGrad, OnNewBuffer, OnDropBuffer, HasModules ...) forward to `self.modules` exactly as they do
// for `OpenCL<Mods>`; custos generates them for its own devices with the macros below.
custos::impl_device_traits!(HIP);
custos::impl_retriever!(HIP);
custos::impl_buffer_hook_traits!(HIP);
custos::pass_down_grad_fn!(HIP);
custos::pass_down_optimize_mem_graph!(HIP);
custos::pass_down_use_gpu_or_cpu!(HIP);
custos::pass_down_replace_buf!(HIP);
