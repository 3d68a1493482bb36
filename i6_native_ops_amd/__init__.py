from ._version import __version__  # noqa: F401
