"""Import alias: the package directory is `server-benchmark_amd/`, which is not a Python
identifier; `import server_benchmark_amd` resolves to it."""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
sys.modules[__name__] = importlib.import_module("server-benchmark_amd")
