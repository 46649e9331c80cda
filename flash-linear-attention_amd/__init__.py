"""MI355X-native gated delta rule (Gated DeltaNet) inference path.

The importable package is ``fla_hip`` inside this directory; this file only makes
``importlib.import_module('flash-linear-attention_amd')`` work from the repository root.
"""
import os as _os
import sys as _sys

_here = _os.path.dirname(_os.path.abspath(__file__))
if _here not in _sys.path:
    _sys.path.insert(0, _here)

import fla_hip  # noqa: E402,F401
from fla_hip import *  # noqa: E402,F401,F403
