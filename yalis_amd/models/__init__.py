"""Architectures.  Importing the package registers the ones it ships."""
from . import llama, nutavik, suranex  # noqa: F401
