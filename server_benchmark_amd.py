"""Import name of the package: its directory is `server-benchmark_amd/`, which is not a Python
identifier, so this module loads that directory's `__init__.py` as the package
`server_benchmark_amd` (submodules resolve inside the directory, under this one name)."""
import importlib.util
import os
import sys

_pkg_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "server-benchmark_amd")
_spec = importlib.util.spec_from_file_location(__name__, os.path.join(_pkg_dir, "__init__.py"),
                                               submodule_search_locations=[_pkg_dir])
_pkg = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _pkg
_spec.loader.exec_module(_pkg)
