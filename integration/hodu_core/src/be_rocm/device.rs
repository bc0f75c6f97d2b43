//! One `RocmDevice` per device id, created on first use and kept in a global map
//! (the shape of be_cuda/device.rs:12-65).
use crate::{
    be::device::BackendDeviceT,
    be_rocm::storage::RocmStorage,
    error::{HoduError, HoduResult},
    types::DType,
};
use hodu_rocm_kernels::Context;
use std::{
    collections::HashMap,
    fmt,
    sync::{Arc, LazyLock, RwLock},
};

#[derive(Clone)]
pub struct RocmDevice {
    pub(crate) id: usize,
    pub(crate) ctx: Arc<Context>,
}

static ROCM_DEVICES: LazyLock<RwLock<HashMap<usize, Arc<RocmDevice>>>> = LazyLock::new(|| RwLock::new(HashMap::new()));

impl fmt::Debug for RocmDevice {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "RocmDevice({})", self.id)
    }
}

impl RocmDevice {
    pub fn get(id: usize) -> HoduResult<Arc<RocmDevice>> {
        if let Some(dev) = ROCM_DEVICES.read()?.get(&id) {
            return Ok(dev.clone());
        }
        let mut devices = ROCM_DEVICES.write()?;
        if let Some(dev) = devices.get(&id) {
            return Ok(dev.clone());
        }
        let ctx = Context::new(id).map_err(|e| HoduError::BackendError(format!("ROCm device {id}: {e}")))?;
        let dev = Arc::new(RocmDevice { id, ctx });
        devices.insert(id, dev.clone());
        Ok(dev)
    }
    pub fn global() -> HoduResult<Arc<RocmDevice>> {
        Self::get(0)
    }
    pub fn context(&self) -> &Arc<Context> {
        &self.ctx
    }
}

impl BackendDeviceT for RocmDevice {
    type BackendStorage = RocmStorage;

    /// uninitialised, as on the CPU (be_cpu/device.rs:19-24): every kernel writes all of its output
    fn allocate(size: usize, dtype: DType) -> HoduResult<RocmStorage> {
        let dev = RocmDevice::global()?;
        let buf = dev.ctx.alloc(size * dtype.size_in_bytes())?;
        Ok(RocmStorage::plain(dev, Arc::new(buf), dtype, size))
    }
    // tensors are created on the CPU and uploaded (be/device.rs:73-143), as for CUDA (be_cuda/device.rs:191-201)
    fn zeros(_: usize, _: DType) -> HoduResult<RocmStorage> {
        Err(HoduError::NotImplemented("RocmDevice::zeros: create on the CPU, then to_device".into()))
    }
    fn randn(_: usize, _: DType, _: f32, _: f32) -> HoduResult<RocmStorage> {
        Err(HoduError::NotImplemented("RocmDevice::randn: create on the CPU, then to_device".into()))
    }
    fn rand_uniform(_: usize, _: DType, _: f32, _: f32) -> HoduResult<RocmStorage> {
        Err(HoduError::NotImplemented("RocmDevice::rand_uniform: create on the CPU, then to_device".into()))
    }
}
