"""Importing this package registers every architecture the engine serves."""
from . import bumolix, dafotar, gemma2, pubunex, rotalorn  # noqa: F401
