"""The transcript byte layout restated in Python from its written definition:

    state_0        = H(label padded with zeros to 32 bytes)
    state_{k+1}    = H(state_k || 28 zero bytes || be32(k) || payload)
    append_message : payload = label padded with zeros to 32 bytes
    append_u64     : payload = 24 zero bytes || be64(x)
    append_scalar  : payload = be64(c1) || be64(c0)
    append_scalars : append_message("begin_append_vector"), each scalar, append_message("end_append_vector")
    challenge      : empty payload; c0 = le64(state[0:8]) mod p, c1 = le64(state[8:16]) mod p

H is BLAKE3; it is passed in so that the layout is checked separately from the hash."""
from pyfield import P


class PyTranscript:
    def __init__(self, H, label=b"m2vec"):
        self.H = H
        self.state = H(label.ljust(32, b"\0"))
        self.k = 0

    def _absorb(self, payload):
        self.state = self.H(self.state + b"\0" * 28 + self.k.to_bytes(4, "big") + payload)
        self.k += 1

    def append_message(self, label):
        self._absorb(label.ljust(32, b"\0"))

    def append_bytes(self, data):
        self._absorb(data)

    def append_u64(self, x):
        self._absorb(b"\0" * 24 + x.to_bytes(8, "big"))

    def append_scalar(self, x):
        self._absorb(int(x[1]).to_bytes(8, "big") + int(x[0]).to_bytes(8, "big"))

    def append_scalars(self, xs):
        self.append_message(b"begin_append_vector")
        for x in xs:
            self.append_scalar(x)
        self.append_message(b"end_append_vector")

    def challenge_scalar(self):
        self._absorb(b"")
        return (int.from_bytes(self.state[0:8], "little") % P, int.from_bytes(self.state[8:16], "little") % P)

    def append_and_sample(self, label):
        self.append_message(label)
        return self.challenge_scalar()
