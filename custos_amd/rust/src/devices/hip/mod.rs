//! The `HIP` device: custos' element-wise path on AMD Instinct GPUs through `libcustos_hip.so`.
//!
//! Laid out like `src/devices/cuda/` (`mod.rs:1-42`): a device type that plugs into the module
//! stack (`hip.rs`), its state (`hip_device.rs`), the pointer type of its buffers (`hip_ptr.rs`),
//! the operation traits (`ops.rs`), unary fusing (`fusing.rs`) and the lazy-run hooks (`lazy.rs`).
//! Kernels are not formatted here: an expression crosses the C ABI as the text `ToCLSource`
//! prints, and the library turns it into a vectorised kernel for the device's architecture.
//!
//! To add it to custos: copy this directory to `src/devices/hip/`, add `pub mod hip;` next to
//! `pub mod cuda;` in `src/devices/mod.rs`, `hip = ["std"]` to `[features]`, the re-exports
//! `pub use devices::hip::HIP;` in `src/lib.rs`, and the link lines to `build.rs`.

pub mod api;

mod fusing;
mod hip;
mod hip_device;
mod hip_ptr;
#[cfg(feature = "lazy")]
pub mod lazy;
mod ops;

pub use hip::*;
pub use hip_device::*;
pub use hip_ptr::*;
pub use ops::*;

/// A buffer of the `HIP` device (as `CUBuffer`, `src/devices/cuda/mod.rs:33`).
pub type HipBuffer<T> = HipPtr<T>;

/// The device index from `CUSTOS_HIP_DEVICE_IDX`, 0 if unset
/// (`chosen_cu_idx`, `src/devices/cuda/mod.rs:35-42`).
pub fn chosen_hip_idx() -> usize {
    let idx = unsafe { api::custos_hip_chosen_device_idx() };
    assert!(
        idx >= 0,
        "Environment variable 'CUSTOS_HIP_DEVICE_IDX' contains an invalid HIP device index!"
    );
    idx as usize
}

/// Element types the library computes in, by the `custos_hip_dtype` number of `T`.
/// `half::f16` / `half::bf16` map to the types that round every node of an expression to 16 bits
/// (12, 13), which is the arithmetic of the `half` crate (`src/number.rs:487-676`); the
/// library's plain 16-bit types (4, 5) compute a whole expression in `f32` and round once at
/// the store.
pub trait HipDatatype: crate::CDatatype {
    const HIP_DTYPE: i32;
}

macro_rules! impl_hip_datatype {
    ($($t:ty => $id:expr),*) => {
        $(impl HipDatatype for $t { const HIP_DTYPE: i32 = $id; })*
    };
}

impl_hip_datatype!(
    f32 => 0, f64 => 1, i32 => 2, i64 => 3, u8 => 6, i8 => 7, i16 => 8, u16 => 9, u32 => 10, u64 => 11
);
#[cfg(feature = "half")]
impl_hip_datatype!(half::f16 => 12, half::bf16 => 13);

/// The `custos_hip_dtype` number of `T` if the library computes in it (`unary_fuse_op` is
/// declared for every `CDatatype`, `src/devices/fusing.rs:21-35`, so it asks at run time).
pub fn dtype_of<T: 'static>() -> Option<i32> {
    use core::any::TypeId;
    let id = TypeId::of::<T>();
    let known: [(TypeId, i32); 10] = [
        (TypeId::of::<f32>(), 0),
        (TypeId::of::<f64>(), 1),
        (TypeId::of::<i32>(), 2),
        (TypeId::of::<i64>(), 3),
        (TypeId::of::<u8>(), 6),
        (TypeId::of::<i8>(), 7),
        (TypeId::of::<i16>(), 8),
        (TypeId::of::<u16>(), 9),
        (TypeId::of::<u32>(), 10),
        (TypeId::of::<u64>(), 11),
    ];
    if let Some((_, dtype)) = known.iter().find(|(t, _)| *t == id) {
        return Some(*dtype);
    }
    #[cfg(feature = "half")]
    {
        if id == TypeId::of::<half::f16>() {
            return Some(12);
        }
        if id == TypeId::of::<half::bf16>() {
            return Some(13);
        }
    }
    None
}
