"""Configuration errors (veloxquant_mlx/core/exceptions.py:12 in the reference)."""


class QuantizerConfigError(ValueError):
    """Raised when a quantizer or cache is configured with invalid values."""
