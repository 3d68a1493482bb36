"""Version of the package: what setup.py installs it under and what the modules report as ``__version__``
(the reference's modules report the version of the installed distribution, fbw/__init__.py:8)."""
__version__ = "0.3.0"
