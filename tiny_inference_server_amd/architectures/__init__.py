"""Architectures: each module turns its configuration into a spec of parts and registers itself."""
from . import fesupel, fikevik, fipuzen, gqa_mtp, rurorax  # noqa: F401  (registration)
