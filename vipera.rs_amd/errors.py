"""Typed errors with the exit codes of the command line.

Kinds and codes follow the reference's error type
(crates/vipera-errors/src/lib.rs:12-47, 94-104): usage 1, bad input 2,
infeasible 3, internal 4.
"""


class ViperaError(Exception):
    """Base of every error this package raises on purpose."""

    exit_code = 4
    kind = "internal"


class UsageError(ViperaError):
    exit_code = 1
    kind = "usage"


class IoError(ViperaError):
    exit_code = 2
    kind = "io"


class ParseError(ViperaError):
    exit_code = 2
    kind = "parse"


class UnsupportedError(ViperaError):
    exit_code = 2
    kind = "unsupported"


class InvalidArgumentError(ViperaError):
    exit_code = 2
    kind = "invalid argument"


class InfeasibleError(ViperaError):
    exit_code = 3
    kind = "infeasible"


class InternalError(ViperaError):
    exit_code = 4
    kind = "internal"
