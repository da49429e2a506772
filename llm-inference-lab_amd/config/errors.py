"""Error types raised while reading configurations and weights."""


class ConfigError(ValueError):
    """A configuration key is missing, of the wrong type, or not supported."""


class WeightError(ValueError):
    """The tensors of a model file do not match what the model expects.

    Raised once per load with every problem found: ``missing`` names,
    ``unexpected`` names, and ``wrong_shape`` entries (name, expected, found)."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)


class UnsupportedSizeError(ValueError):
    """A kernel was asked for a size it does not take (it refuses rather than
    computing a wrong result)."""
