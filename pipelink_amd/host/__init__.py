from .backend import HipBackend, PlkError, load_library  # noqa: F401
