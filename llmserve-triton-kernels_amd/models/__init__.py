"""Architectures: each module registers a name, a configuration class and a spec builder."""

from . import dibepel, felavik, llama, milozen, nolavik  # noqa: F401
