use core::ops::{Deref, DerefMut};

use crate::{
    Alloc, Base, Buffer, CloneBuf, Device, IsShapeIndep, Module as CombModule, OnNewBuffer, Setup, Shape, Unit,
    WrappedData, flag::AllocFlag, impl_device_traits,
};

use super::{
    AsHipKernelArg, HipDevice, HipPtr,
    api::{custos_hip_copy, custos_hip_write},
};

pub trait IsHip: Device {}

/// Used to perform calculations on an AMD GPU through `libcustos_hip.so`.
/// Takes the place of `CUDA<Mods>` (`src/devices/cuda/cuda.rs:22-25`): same fields, same
/// module stack, same traits, so `CUDA<Lazy<Graph<Base>>>` becomes `HIP<Lazy<Graph<Base>>>`.
pub struct HIP<Mods = Base> {
    pub modules: Mods,
    pub device: HipDevice,
}

impl_device_traits!(HIP);

impl<Mods> Deref for HIP<Mods> {
    type Target = HipDevice;

    #[inline]
    fn deref(&self) -> &Self::Target {
        &self.device
    }
}

impl<Mods> DerefMut for HIP<Mods> {
    #[inline]
    fn deref_mut(&mut self) -> &mut Self::Target {
        &mut self.device
    }
}

impl<SimpleMods> HIP<SimpleMods> {
    /// Returns a [HIP] device at the specified device index.
    /// # Errors
    /// - No device was found at the given device index
    /// - some other HIP related errors
    #[inline]
    pub fn new<'a, NewMods>(idx: usize) -> crate::Result<HIP<NewMods>>
    where
        Self: 'a,
        SimpleMods: CombModule<'a, HIP, Module = NewMods>,
        NewMods: Setup<HIP<NewMods>>,
    {
        let mut hip = HIP { modules: SimpleMods::new(), device: HipDevice::new(idx)? };
        NewMods::setup(&mut hip)?;
        Ok(hip)
    }
}

impl<Mods: WrappedData> Device for HIP<Mods> {
    type Data<'a, T: Unit, S: Shape> = Mods::Wrap<'a, T, HipPtr<T>>;
    type Base<T: Unit, S: Shape> = HipPtr<T>;
    type Error = i32;

    #[inline(always)]
    fn default_base_to_data<'a, T: Unit, S: Shape>(&'a self, base: Self::Base<T, S>) -> Self::Data<'a, T, S> {
        self.wrap_in_base(base)
    }

    #[inline(always)]
    fn default_base_to_data_unbound<'a, T: Unit, S: Shape>(&self, base: Self::Base<T, S>) -> Self::Data<'a, T, S> {
        self.wrap_in_base_unbound(base)
    }

    #[inline(always)]
    fn wrap_to_data<'a, T: Unit, S: Shape>(&self, wrap: Self::Wrap<'a, T, Self::Base<T, S>>) -> Self::Data<'a, T, S> {
        wrap
    }

    #[inline(always)]
    fn data_as_wrap<'a, 'b, T: Unit, S: Shape>(
        data: &'b Self::Data<'a, T, S>,
    ) -> &'b Self::Wrap<'a, T, Self::Base<T, S>> {
        data
    }

    #[inline(always)]
    fn data_as_wrap_mut<'a, 'b, T: Unit, S: Shape>(
        data: &'b mut Self::Data<'a, T, S>,
    ) -> &'b mut Self::Wrap<'a, T, Self::Base<T, S>> {
        data
    }
}

impl<Mods: WrappedData, T: Unit> Alloc<T> for HIP<Mods> {
    /// Zero-filled, like the CPU device (gradients rely on it); the CUDA device hands out
    /// uninitialised memory (`src/devices/cuda/cuda.rs:114-122`).
    #[inline]
    fn alloc<S: Shape>(&self, len: usize, flag: AllocFlag) -> crate::Result<Self::Base<T, S>> {
        Ok(HipPtr::new(self.handle, len, flag)?)
    }

    fn alloc_from_slice<S: Shape>(&self, data: &[T]) -> crate::Result<Self::Base<T, S>>
    where
        T: Clone,
    {
        let ptr = HipPtr::new(self.handle, data.len(), AllocFlag::None)?;
        // the host range may be reused as soon as the call returns
        self.check(unsafe {
            custos_hip_write(self.handle, ptr.ptr, data.as_ptr().cast(), core::mem::size_of_val(data))
        })?;
        Ok(ptr)
    }
}

unsafe impl<Mods: WrappedData> IsShapeIndep for HIP<Mods> {}

impl<Mods: WrappedData> IsHip for HIP<Mods> {}

#[cfg(feature = "fork")]
impl<Mods> crate::ForkSetup for HIP<Mods> {
    #[inline]
    fn fork_setup(&mut self) {}
}

impl<'a, Mods: WrappedData + OnNewBuffer<'a, T, Self, ()>, T: Unit> CloneBuf<'a, T> for HIP<Mods> {
    fn clone_buf(&'a self, buf: &Buffer<'a, T, HIP<Mods>>) -> Buffer<'a, T, HIP<Mods>> {
        let cloned = Buffer::new(self, buf.len());
        self.check(unsafe {
            custos_hip_copy(self.handle, cloned.hip_ptr(), buf.hip_ptr(), buf.len() * core::mem::size_of::<T>())
        })
        .unwrap();
        cloned
    }
}

impl<'a, Mods: WrappedData, T: Unit> Buffer<'a, T, HIP<Mods>> {
    /// Returns a non null device address (`Buffer::cu_ptr`, `src/buffer.rs:572-583`).
    #[inline]
    pub fn hip_ptr(&self) -> u64 {
        assert!(self.base().ptr != 0, "called hip_ptr() on an invalid HIP buffer");
        self.base().ptr
    }
}

// Buffers as arguments of caller-written kernels (`src/devices/cuda/kernel_launch.rs:47-64`).
impl<'a, T: Unit, Mods: WrappedData, S: Shape> AsHipKernelArg for &Buffer<'a, T, HIP<Mods>, S> {
    #[inline]
    fn as_kernel_arg(&self) -> (*mut core::ffi::c_void, usize) {
        (&self.base().ptr as *const u64 as *mut core::ffi::c_void, 8)
    }
}

impl<'a, T: Unit, Mods: WrappedData, S: Shape> AsHipKernelArg for Buffer<'a, T, HIP<Mods>, S> {
    #[inline]
    fn as_kernel_arg(&self) -> (*mut core::ffi::c_void, usize) {
        (&self.base().ptr as *const u64 as *mut core::ffi::c_void, 8)
    }
}
