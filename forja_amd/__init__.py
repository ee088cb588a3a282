"""forja_amd: MI355X (gfx950) backend for forja's ragged continuous-batch forward step.

`forja_amd.core` holds the contract types, `forja_amd.hip_backend` the binding of the C ABI in
include/forja_hip.h, `forja_amd.build` compiles csrc/ into libforja_hip.so.
"""
from .core import *  # noqa: F401,F403
