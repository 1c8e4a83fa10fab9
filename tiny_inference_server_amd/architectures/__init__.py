"""Architectures: each module turns its configuration into a spec of parts and registers itself."""
from . import gqa_mtp  # noqa: F401  (registration)
