from . import minicpm4  # noqa: F401
