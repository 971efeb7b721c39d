"""Architectures.  Importing this package registers each of them."""

from tokamak_amd.models import qwen3  # noqa: F401
