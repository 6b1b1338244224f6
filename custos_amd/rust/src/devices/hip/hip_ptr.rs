use core::marker::PhantomData;

use super::api::{ALLOC_ZEROED, HipDeviceHandle, custos_hip_alloc, custos_hip_free, custos_hip_read};
use super::{HipResult, check};
use crate::{HasId, Id, PtrType, ShallowCopy, ToDim, Unit, flag::AllocFlag};

/// The pointer used for `HIP` [`Buffer`](crate::Buffer)s (`CUDAPtr`, `src/devices/cuda/cuda_ptr.rs:5-15`).
/// It remembers the library handle it was allocated from: freeing returns the block to that
/// device's pool.
#[derive(Debug, PartialEq, Eq)]
pub struct HipPtr<T> {
    /// Device address.
    pub ptr: u64,
    /// The number of elements addressable.
    pub len: usize,
    /// Allocation flag for the pointer.
    pub flag: AllocFlag,
    pub dev: *mut HipDeviceHandle,
    pub p: PhantomData<T>,
}

unsafe impl<T: Sync> Sync for HipPtr<T> {}
unsafe impl<T: Send> Send for HipPtr<T> {}

impl<T> HipPtr<T> {
    /// A zero-filled allocation of `len` elements, like the CPU device's `alloc`
    /// (`src/devices/cpu/cpu_device.rs:133-145`); a length of 0 is an error
    /// (`src/devices/cuda/api/cuda.rs:69-71`).
    pub fn new(dev: *mut HipDeviceHandle, len: usize, flag: AllocFlag) -> HipResult<Self> {
        let mut ptr = 0u64;
        check(dev, unsafe { custos_hip_alloc(dev, len * core::mem::size_of::<T>(), ALLOC_ZEROED, &mut ptr) })?;
        Ok(HipPtr { ptr, len, flag, dev, p: PhantomData })
    }

    /// Waits for the compute stream, then copies the elements to the host.
    pub fn read(&self) -> Vec<T>
    where
        T: Default + Clone,
    {
        let mut data = vec![T::default(); self.len];
        let code = unsafe {
            custos_hip_read(self.dev, data.as_mut_ptr().cast(), self.ptr, self.len * core::mem::size_of::<T>())
        };
        assert_eq!(code, 0, "reading a HIP buffer failed");
        data
    }
}

impl<T> HasId for HipPtr<T> {
    #[inline]
    fn id(&self) -> Id {
        Id { id: self.ptr, len: self.len }
    }
}

impl<T> Default for HipPtr<T> {
    #[inline]
    fn default() -> Self {
        Self { ptr: 0, len: 0, flag: AllocFlag::default(), dev: core::ptr::null_mut(), p: PhantomData }
    }
}

impl<T> Drop for HipPtr<T> {
    fn drop(&mut self) {
        if !self.flag.continue_deallocation() || self.ptr == 0 {
            return;
        }
        unsafe { custos_hip_free(self.dev, self.ptr) };
    }
}

impl<T> ShallowCopy for HipPtr<T> {
    #[inline]
    unsafe fn shallow(&self) -> Self {
        HipPtr { ptr: self.ptr, len: self.len, flag: AllocFlag::Wrapper, dev: self.dev, p: PhantomData }
    }
}

impl<T: Unit> PtrType for HipPtr<T> {
    #[inline]
    fn size(&self) -> usize {
        self.len
    }

    #[inline]
    fn flag(&self) -> AllocFlag {
        self.flag
    }

    #[inline]
    unsafe fn set_flag(&mut self, flag: AllocFlag) {
        self.flag = flag;
    }
}

impl<T> ToDim for HipPtr<T> {
    type Out = Self;

    #[inline]
    fn to_dim(self) -> Self::Out {
        self
    }

    #[inline]
    fn as_dim(&self) -> &Self::Out {
        self
    }
}

/// Serialisation as a sequence of elements, like every other pointer type of custos
/// (`src/devices/cuda/cuda_ptr.rs:121-157`).  A pointer has to name a device, so a
/// deserialised one belongs to the device the thread created last (`HIP::new`).
#[cfg(feature = "serde")]
mod serde {
    use super::HipPtr;
    use crate::{
        cpu::CPUPtr,
        flag::AllocFlag,
        hip::{api::custos_hip_write, check, current_handle},
    };
    use core::marker::PhantomData;

    impl<T: serde::Serialize + Default + Clone> serde::Serialize for HipPtr<T> {
        #[inline]
        fn serialize<S: serde::Serializer>(&self, serializer: S) -> Result<S::Ok, S::Error> {
            serializer.collect_seq(self.read().iter())
        }
    }

    impl<'a, T: serde::Deserialize<'a>> serde::Deserialize<'a> for HipPtr<T> {
        fn deserialize<D: serde::Deserializer<'a>>(deserializer: D) -> Result<Self, D::Error> {
            use serde::de::Error;
            let cpu_ptr: CPUPtr<T> = deserializer.deserialize_seq(crate::cpu::serde::CpuPtrVisitor { marker: PhantomData::<T> })?;
            let dev = current_handle().ok_or_else(|| D::Error::custom("no HIP device was created on this thread"))?;
            let ptr = HipPtr::new(dev, cpu_ptr.len, AllocFlag::None).map_err(D::Error::custom)?;
            let bytes = cpu_ptr.len * core::mem::size_of::<T>();
            check(dev, unsafe { custos_hip_write(dev, ptr.ptr, cpu_ptr.ptr.cast(), bytes) }).map_err(D::Error::custom)?;
            Ok(ptr)
        }
    }
}
