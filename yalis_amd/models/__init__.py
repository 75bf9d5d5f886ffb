"""Architectures.  Importing the package registers the ones it ships."""
from . import bekedra, llama, mesolix, nutavik, suranex  # noqa: F401
