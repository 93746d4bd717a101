"""Why a ``.chr`` file was refused.  One class per failure the container format names
(``docs/spec/chr0.md`` appendix B, ``gpu/chr0/errors.py:23-55``), all under ``Chr0Error``."""

from __future__ import annotations

__all__ = ["Chr0Error", "TruncatedError", "HeaderError", "AlignmentError", "SizeMismatchError",
           "OverlapError", "CodecError", "GroupSizeError", "TensorNotFoundError"]


class Chr0Error(Exception):
    """Any rejection of a ``.chr`` file."""


class TruncatedError(Chr0Error):
    """The file ends before its header or one of its byte ranges does."""


class HeaderError(Chr0Error):
    """The length word or the JSON header breaks the format."""


class AlignmentError(Chr0Error):
    """A byte range does not start on a 64-byte boundary."""


class SizeMismatchError(Chr0Error):
    """A byte range is not as long as shape and codec say."""


class OverlapError(Chr0Error):
    """Two byte ranges share bytes."""


class CodecError(Chr0Error):
    """Unknown codec, wrong keys for the codec, or codecs mixed in one file."""


class GroupSizeError(Chr0Error):
    """``group_size`` is not the codec's fixed value."""


class TensorNotFoundError(Chr0Error):
    """The file has no tensor of that name."""
