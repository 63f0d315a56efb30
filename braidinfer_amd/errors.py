"""Typed errors of the library.

The reference has one error enum for the model path (`ModelError`: `MissingWeight`,
`InvalidConfig`, ..., crates/braidinfer-runtime/src/weights.rs:229-268) and panics on
shape mismatches (weights.rs:301-307).  Here every failure a caller can cause is a
Python exception of its own, and none of them is a panic.
"""


class BraidError(Exception):
    """Base class of every error raised by this library."""


class ConfigError(BraidError):
    """config.json is missing a key, holds a bad value, or names an unknown architecture."""


class WeightError(BraidError):
    """The tensors of a model folder do not match what the model needs.

    One error lists everything at once: `missing`, `unexpected` and `mismatched`
    (name, expected shape/dtype, found shape/dtype).
    """

    def __init__(self, message, missing=(), unexpected=(), mismatched=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.mismatched = list(mismatched)


class CacheError(BraidError):
    """A cache request that cannot be served: no free slot or page, a slot used after
    it was freed, freed twice, or never allocated."""


class KernelError(BraidError):
    """A kernel was asked for a size or layout it does not take, or the compiled
    extension is missing."""


class StepError(BraidError):
    """A step's entries do not form a legal batch."""
