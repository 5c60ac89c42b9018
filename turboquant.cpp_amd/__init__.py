"""A small model library with generation of its own for one GPU (gfx950): everything between a request's
tokens and its next token.

``Model`` is the Python entry point, ``python -m turboquant_cpp_amd`` (``cli.py``) the command line, and
``bin/trace_run`` replays given tokens step by step.
"""
from . import config, parts, models  # noqa: F401  (importing registers parts and architectures)
from .api import ChatContextOverflow, Model, load  # noqa: F401

__version__ = "0.3.0"
