from .fmmv import fdmmv, fmmv  # noqa: F401
