"""Architectures.  Importing this package registers each of them."""

from tokamak_amd.models import gubanex, mepupel, qwen3, rorosun, supinex  # noqa: F401
