//! `#[serde(with = "...")]` module for vectors of field elements, in the place of the
//! `dp_crypto::serialization` the reference's proof structs name
//! (`zkml/src/layers/einsum/mod.rs:588-599`, `zkml/src/lookup/logup_gkr/structs.rs:561-578`).
//! Encoding: one byte string, 16 bytes per element, `c0` then `c1`, each little-endian.  dp-crypto's own
//! bytes (ark-serialize of its field) are not known here, and its field is not this one: a proof made
//! with this engine is read back by this module, not by dp-crypto's.

use serde::de::Error as _;
use serde::{Deserialize, Deserializer, Serializer};

use crate::field::ExtField;

pub fn serialize<F: ExtField, S: Serializer>(xs: &[F], s: S) -> Result<S::Ok, S::Error> {
    let mut bytes = Vec::with_capacity(16 * xs.len());
    for x in xs {
        let l = x.to_limbs();
        bytes.extend_from_slice(&l[0].to_le_bytes());
        bytes.extend_from_slice(&l[1].to_le_bytes());
    }
    s.serialize_bytes(&bytes)
}

pub fn deserialize<'de, F: ExtField, D: Deserializer<'de>>(d: D) -> Result<Vec<F>, D::Error> {
    let bytes: Vec<u8> = Vec::<u8>::deserialize(d)?;
    if bytes.len() % 16 != 0 {
        return Err(D::Error::custom("field vector: length is not a multiple of 16 bytes"));
    }
    let mut out = Vec::with_capacity(bytes.len() / 16);
    for c in bytes.chunks_exact(16) {
        let c0 = u64::from_le_bytes(c[..8].try_into().expect("8 bytes"));
        let c1 = u64::from_le_bytes(c[8..].try_into().expect("8 bytes"));
        out.push(F::from_limbs(c0, c1).ok_or_else(|| D::Error::custom("field vector: limb not canonical"))?);
    }
    Ok(out)
}
