"""mference_amd — MI355X-native MoE expert hot path of Mference (libmfmoe + host mirror)."""
from ._capi import LIB_PATH, LibraryMissing, MfError  # noqa: F401

__version__ = "0.1.0"
