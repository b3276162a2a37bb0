"""C++ host layer of the compressed multiply path, exposed to Python.

`systemds_amd.host.load()` returns the compiled module `_clahost` (built by
`systemds_amd.build.build_host`); it links against libclahip.so and has no CPU
compute path of its own.
"""
import importlib
import os


def load():
    here = os.path.dirname(os.path.abspath(__file__))
    if not os.path.exists(os.path.join(here, "_clahost.so")):
        raise ImportError("systemds_amd/host/_clahost.so is not built: run python -m systemds_amd.build")
    return importlib.import_module("systemds_amd.host._clahost")
