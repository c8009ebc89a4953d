//! One GPU context: a HIP stream and a device memory pool (`dps_ctx_create`).  Calls on one context
//! must not overlap; give every proving thread a context of its own (the reference proves chunks
//! from a thread pool, `zkml/src/graph/executor.rs:148`): the library shares the GPU between them.

use std::ffi::CStr;
use std::ptr;
use std::rc::Rc;

use dp_sumcheck_sys as sys;

use crate::error::{Error, Result};

struct Raw(*mut sys::dps_ctx);

impl Drop for Raw {
    fn drop(&mut self) {
        unsafe {
            sys::dps_ctx_destroy(self.0);
        }
    }
}

/// Cheap to clone; the context is destroyed when the last clone and the last table made from it go.
/// Neither `Send` nor `Sync`: a context and the tables made from it stay on the thread that created
/// them, which is what keeps calls on one context from overlapping.
#[derive(Clone)]
pub struct Context {
    raw: Rc<Raw>,
}

impl Context {
    pub fn new(device: i32) -> Result<Self> {
        let mut h: *mut sys::dps_ctx = ptr::null_mut();
        let rc = unsafe { sys::dps_ctx_create(device, &mut h) };
        if rc != sys::DPS_OK {
            return Err(Error { status: rc, message: format!("dps_ctx_create: {}", status_text(rc)) });
        }
        Ok(Context { raw: Rc::new(Raw(h)) })
    }

    pub fn as_ptr(&self) -> *mut sys::dps_ctx {
        self.raw.0
    }

    /// Waits for everything queued on the context's stream.
    pub fn sync(&self) -> Result<()> {
        let rc = unsafe { sys::dps_ctx_sync(self.as_ptr()) };
        self.check(rc, "dps_ctx_sync")
    }

    pub(crate) fn check(&self, rc: i32, what: &str) -> Result<()> {
        if rc == sys::DPS_OK {
            return Ok(());
        }
        let detail = unsafe { CStr::from_ptr(sys::dps_last_error(self.as_ptr())) }.to_string_lossy().into_owned();
        Err(Error { status: rc, message: format!("{}: {} ({})", what, status_text(rc), detail) })
    }
}

/// Cap, in compute units, on what the launches that wait on the GPU of all contexts of this process may
/// hold on `device` together (`-1`: the whole device, `0`: nothing ever waits there).
pub fn set_resident_budget(device: i32, compute_units: i32) -> Result<()> {
    let rc = unsafe { sys::dps_device_set_resident_budget(device, compute_units) };
    if rc == sys::DPS_OK {
        Ok(())
    } else {
        Err(Error { status: rc, message: format!("dps_device_set_resident_budget: {}", status_text(rc)) })
    }
}

pub(crate) fn status_text(rc: i32) -> String {
    unsafe { CStr::from_ptr(sys::dps_status_str(rc)) }.to_string_lossy().into_owned()
}
