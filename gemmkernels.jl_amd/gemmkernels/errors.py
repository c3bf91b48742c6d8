"""Exceptions of the host layer."""


class ConfigError(Exception):
    """reference src/config.jl:78-82.  ``status`` is the gk_status of the C ABI when the error
    came from the library."""

    def __init__(self, message: str, status: int = 0):
        super().__init__(message)
        self.message = message
        self.status = status

    def __str__(self):
        return f"ConfigError: {self.message}"


class DimensionMismatch(Exception):
    """Julia's DimensionMismatch as thrown by create_config (reference src/matmul.jl:75-77)."""
