//! The Fiat-Shamir interface the engine needs of the caller's transcript.  The transcript itself is
//! the caller's (in the reference: dp-crypto's `Blake3Transcript`, `zkml/src/lib.rs:106-108`), lives
//! on the host and is threaded through `prove` by `&mut`; the GPU never sees it.  The method set is the
//! one the layer provers use (`zkml/src/layers/einsum/prove.rs:158,278`,
//! `zkml/src/lookup/logup_gkr/prover.rs:163-173,261,284-288`, `zkml/src/lib.rs:176-184`).

use crate::field::ExtField;

pub trait Transcript<F: ExtField> {
    fn append_scalars(&mut self, xs: &[F]);
    fn challenge_scalar(&mut self) -> F;
    fn append_bytes(&mut self, data: &[u8]);
    fn append_message(&mut self, label: &'static [u8]);
    fn append_u64(&mut self, x: u64);

    fn append_and_sample(&mut self, label: &'static [u8]) -> F {
        self.append_message(label);
        self.challenge_scalar()
    }
    /// `VectorTranscript::read_challenges`
    fn read_challenges(&mut self, n: usize) -> Vec<F> {
        (0..n).map(|_| self.challenge_scalar()).collect()
    }
}
