"""Error types of the host layer, one per variant the reference's op API can return on this path
(singe-kernel/src/error.rs:12-186; singe/src/error/mod.rs for IndexOutOfBounds / InvalidArgument)."""
from __future__ import annotations


class Error(Exception):
    """Base of every failure raised by the attention host layer."""


class InvalidLength(Error):
    """A logical length is invalid for the requested operation (Error::InvalidLength)."""


class LengthTooShort(Error):
    """A named buffer has fewer elements than required (Error::LengthTooShort)."""

    def __init__(self, name: str, minimum: int, actual: int):
        super().__init__(f"length too short for {name}: minimum {minimum}, actual {actual}")
        self.name, self.minimum, self.actual = name, minimum, actual


class LengthMismatch(Error):
    """Two extents that must agree differ (Error::LengthMismatch)."""


class LengthExceedsI32(Error):
    """A dimension cannot fit the native signed 32-bit interface (Error::LengthExceedsI32)."""


class SizeOverflow(Error):
    """Checked size arithmetic overflowed (Error::SizeOverflow)."""


class UnsupportedWidth(Error):
    """The operation does not support the requested width (Error::UnsupportedWidth)."""

    def __init__(self, op: str, width: int):
        super().__init__(f"unsupported width for {op}: width = {width}")
        self.op, self.width = op, width


class NullPointer(Error):
    """A required device pointer is null (Error::NullPointer)."""


class KernelNotPrepared(Error):
    """The code object is missing or cannot be loaded (Error::KernelNotPrepared)."""


class UnsupportedConfiguration(Error):
    """The operation cannot execute this combination of settings (Error::UnsupportedConfiguration)."""


class InvalidArgument(Error):
    """Shapes or types break the op's rules (singe::Error::InvalidArgument)."""


class IndexOutOfBounds(Error):
    """A paging value addresses outside its buffers (singe::Error::IndexOutOfBounds)."""


class TuneCacheMiss(Error):
    """TuningChoice::Cached found no cached entry (Error::TuneCacheMiss)."""


class AutotuneDuringCapture(Error):
    """Candidates cannot be timed while the stream is being captured (Error::AutotuneDuringCapture)."""


class NoTuneCandidates(Error):
    """No candidate is left to time, or none completed (Error::NoTuneCandidates / NoSuccessfulTuneCandidates)."""


class StaleRecord(Error):
    """singe::Error::StaleRecord: parameters a kernel does not take (any more)."""


class Hip(Error):
    """A HIP runtime call failed (the counterpart of Error::Cuda)."""

    def __init__(self, code: int, message: str, what: str):
        super().__init__(f"hip error {code} in {what}: {message}")
        self.code = code
