"""webgpt_amd: MI355X (gfx950) implementation of WebGPT's per-token transformer
forward path behind the reference's GPT / instruction-block interface.

Host side of the C ABI declared in include/webgpt_amd.h. Importing this package
does not need a GPU; any compute call does, and raises if the shared library or
the device is missing.
"""
from . import _lib  # noqa: F401
from ._lib import WgptError  # noqa: F401
