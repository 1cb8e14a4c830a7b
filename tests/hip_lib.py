"""Loads the package's Python binding (allreduce-proto_amd/ibcomm_hip.py) under the name the tests use.
The directory name has a hyphen, so it is loaded by path rather than imported."""
import importlib.util
import os
import sys

_path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "allreduce-proto_amd", "ibcomm_hip.py")
_spec = importlib.util.spec_from_file_location("ibcomm_hip", _path)
_mod = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_mod)
sys.modules[__name__] = _mod
