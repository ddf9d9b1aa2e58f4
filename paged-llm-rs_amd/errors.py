"""The five kinds of failure the engine reports (reference: error.rs:9-22)."""

from __future__ import annotations


class PagedLLMError(Exception):
    """Base of every error this package raises on purpose."""


class TensorError(PagedLLMError):
    """A kernel launch or device call failed, or was given operands it refuses."""


class IoError(PagedLLMError):
    """A file could not be read or written."""


class ConfigError(PagedLLMError):
    """A config file or an argument is invalid or lacks a field."""


class UnsupportedError(PagedLLMError):
    """The config describes a model this implementation would have to
    misinterpret in order to run."""


class WeightError(PagedLLMError):
    """The weight file lacks tensors the model needs, holds some it does not
    know, or holds them at the wrong shape."""
