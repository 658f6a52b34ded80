from . import observer, qconfig, qscheme  # noqa: F401
