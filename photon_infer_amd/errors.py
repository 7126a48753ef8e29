"""Typed errors of the engine.

The reference returns ``Result<T, Error>`` values whose ``ErrorCode`` is grouped by
subsystem (include/photon/core/error.hpp:40-87).  Python raises instead of returning,
so each group becomes an exception class that carries the same code; callers that want
the reference's style can catch ``PhotonError`` and read ``.code``.
"""
from __future__ import annotations

import enum


class ErrorCode(enum.IntEnum):
    """Numeric codes, grouped as in include/photon/core/error.hpp:40-87."""

    OK = 0
    # memory 1-99
    OUT_OF_MEMORY = 1
    BUFFER_OVERFLOW = 4
    # io 100-199
    FILE_NOT_FOUND = 100
    FILE_READ_ERROR = 101
    FILE_WRITE_ERROR = 102
    INVALID_FILE_FORMAT = 103
    # tensor 200-299
    INVALID_SHAPE = 200
    INVALID_DTYPE = 201
    SHAPE_MISMATCH = 202
    DEVICE_MISMATCH = 203
    INVALID_INDEX = 204
    # model 300-399
    MODEL_LOAD_ERROR = 300
    INVALID_MODEL_FORMAT = 301
    UNSUPPORTED_MODEL = 302
    WEIGHT_MISMATCH = 303
    MODEL_PARSE_ERROR = 304
    # operator 400-499
    INVALID_OPERATOR = 400
    OPERATOR_NOT_IMPLEMENTED = 401
    INVALID_OPERAND = 402
    # device 500-599
    DEVICE_ERROR = 500
    KERNEL_LIBRARY_MISSING = 504
    # generic 900-999
    INVALID_ARGUMENT = 900
    NOT_IMPLEMENTED = 901
    INTERNAL_ERROR = 902


class PhotonError(Exception):
    """Base of every error the engine raises on purpose."""

    code: ErrorCode = ErrorCode.INTERNAL_ERROR

    def __init__(self, message: str, code: ErrorCode | None = None):
        super().__init__(message)
        if code is not None:
            self.code = code

    def __str__(self) -> str:  # "[WeightMismatch] ..." like Error::to_string
        return f"[{self.code.name}] {super().__str__()}"


class ConfigError(PhotonError):
    """config.json cannot be parsed or holds a value the engine rejects."""

    code = ErrorCode.MODEL_PARSE_ERROR


class UnsupportedModelError(PhotonError):
    """The architecture, or one of its options, is not one this engine builds."""

    code = ErrorCode.UNSUPPORTED_MODEL


class WeightError(PhotonError):
    """Missing / unexpected tensors or wrong shapes in a model folder."""

    code = ErrorCode.WEIGHT_MISMATCH


class FileFormatError(PhotonError):
    code = ErrorCode.INVALID_FILE_FORMAT


class OutOfPagesError(PhotonError):
    """The page pool of a cache group cannot serve an allocation."""

    code = ErrorCode.OUT_OF_MEMORY


class OutOfMemoryError(PhotonError):
    """Device memory cannot hold what was asked for (the cache pools, a workspace)."""

    code = ErrorCode.OUT_OF_MEMORY


class CacheError(PhotonError):
    """Misuse of the cache manager: double free, unknown request, no free slot."""

    code = ErrorCode.INVALID_ARGUMENT


class KernelError(PhotonError):
    """A kernel refused its operands (size it does not take, wrong dtype, ...)."""

    code = ErrorCode.INVALID_OPERAND


class KernelLibraryMissing(PhotonError):
    """The HIP extension cannot be built or loaded; there is no fallback."""

    code = ErrorCode.KERNEL_LIBRARY_MISSING


class RequestError(PhotonError):
    """A request the engine cannot serve (empty, too long, bad token id)."""

    code = ErrorCode.INVALID_ARGUMENT
