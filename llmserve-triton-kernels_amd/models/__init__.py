"""Architectures: each module registers a name, a configuration class and a spec builder."""

from . import dibepel, llama, milozen  # noqa: F401
