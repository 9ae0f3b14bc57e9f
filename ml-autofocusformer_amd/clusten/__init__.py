"""Drop-in `clusten` package: the three CLUSTEN autograd Functions on gfx950 HIP kernels.

Mirrors clusten/__init__.py:6 of the reference:

    from clusten import CLUSTENQKFunction, CLUSTENAVFunction, CLUSTENWFFunction
"""
from .clusten import CLUSTENQKFunction, CLUSTENAVFunction, CLUSTENWFFunction  # noqa: F401

__all__ = ["CLUSTENQKFunction", "CLUSTENAVFunction", "CLUSTENWFFunction"]
