"""tmq_amd -- MI355X-native implementation of TMQ's GPU hot path behind TMQ's Python API."""
from . import _capi  # noqa: F401
