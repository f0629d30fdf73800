"""Exception types of the pack readers and operators.

Same names and base classes as the reference's (common/errors.py:17-32,
formats/qvb8r/container.py:26-27, formats/qvb8/escape_split.py:37-38), so code that
catches them keeps working.
"""

__all__ = ["Qvb8Error", "UncertifiableTensor", "QVB8RFormatError", "EscapeTableError",
           "NativeLibraryError"]


class Qvb8Error(ValueError):
    """A blob that is not a readable QVB8 / QVBD pack, or a tensor that cannot be
    represented under the requested tau."""


class UncertifiableTensor(Qvb8Error):
    """No storage dtype can hold the certified bound for this tensor."""


class QVB8RFormatError(ValueError):
    """A .qvb8r file that cannot be read (magic, version, crc32, PB)."""


class EscapeTableError(RuntimeError):
    """escape_tables.json is missing, unreadable, or does not match the pack."""


class NativeLibraryError(RuntimeError):
    """The HIP library is missing or a call into it failed.  There is no CPU
    fallback: every operator needs the native library."""
