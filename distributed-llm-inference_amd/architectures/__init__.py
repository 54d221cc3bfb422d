"""Architectures that ship with the engine. Importing this package registers them."""

from . import betepel, llama, makodra, miberax, zarinex  # noqa: F401
