"""Architectures; importing this package registers the built-in ones."""
from . import besulix, gemma2, golepel, lutovik, vogunex   # noqa: F401
