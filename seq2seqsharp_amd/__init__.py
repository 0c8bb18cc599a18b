"""TensorSharp.HIP for MI355X: host-side mirror of the reference interfaces over libtship.so."""
from ._lib import TSHipError, lib  # noqa: F401
