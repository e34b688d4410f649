from . import opt  # noqa: F401
