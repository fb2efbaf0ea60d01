"""Faces of the HIP kernels (see ``kernels.py``) and the library builder (``library.py``)."""
