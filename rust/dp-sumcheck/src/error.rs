//! Status codes of the C ABI as a Rust error.  dp-crypto's `prove` is infallible by panic; the ABI
//! returns a status from every call, and the adapter turns a non-zero one into this.

use std::fmt;

#[derive(Debug, Clone, PartialEq, Eq)]
pub struct Error {
    /// the `dps_status` the library returned
    pub status: i32,
    /// what was being called, the status text, and the context's last error text when there is one
    pub message: String,
}

pub type Result<T> = std::result::Result<T, Error>;

impl Error {
    pub fn invalid(message: impl Into<String>) -> Self {
        Error { status: dp_sumcheck_sys::DPS_ERR_INVALID, message: message.into() }
    }
}

impl fmt::Display for Error {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "[status {}] {}", self.status, self.message)
    }
}

impl std::error::Error for Error {}
