use crate::{HIP, UnaryFusing, WrappedData};

impl<Mods: WrappedData> UnaryFusing for HIP<Mods> {
    /// A chain of unary operations as ONE kernel: the statement list
    /// `x = op_1(x);\nx = op_2(x);\n…` that `operations_to_fused_src` prints
    /// (`src/devices/fusing.rs:4-19`) is a kernel source the library accepts as it is
    /// (`src/devices/cuda/fusing.rs:8-50` wraps the same text into a kernel string).
    #[cfg(feature = "lazy")]
    #[cfg(feature = "graph")]
    #[inline]
    fn unary_fuse_op<T: crate::CDatatype + crate::Numeric>(
        &self,
        ops_to_fuse: Vec<std::rc::Rc<dyn Fn(crate::Resolve<T>) -> Box<dyn crate::TwoWay<T>>>>,
    ) -> Box<dyn Fn((&mut crate::Buffer<'_, T, Self, ()>, &crate::Buffer<'_, T, Self, ()>), &Self) -> crate::Result<()>>
    {
        use super::api::{KIND_APPLY, custos_hip_apply_fn};
        use crate::operations_to_fused_src;

        let dtype = super::dtype_of::<T>();
        Box::new(move |(out, buf), dev| {
            if ops_to_fuse.is_empty() {
                return Ok(());
            }
            let dtype = dtype.ok_or(crate::DeviceError::UnaryFusingUnsupported)?;
            let fused_operations = operations_to_fused_src(&ops_to_fuse);
            let kernel = dev.compile(KIND_APPLY, dtype, &fused_operations, &[c"x"])?;
            dev.check(unsafe { custos_hip_apply_fn(dev.handle, kernel, buf.base().ptr, out.base().ptr, buf.len()) })?;
            Ok(())
        })
    }
}
