"""Import alias: `import fairseq_apollo_amd` loads the package that lives in the
directory `fairseq-apollo_amd/` (a hyphen cannot appear in an import statement)."""
import importlib.util
import os
import sys

_here = os.path.dirname(os.path.abspath(__file__))
_pkg = os.path.join(_here, "fairseq-apollo_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_pkg, "__init__.py"), submodule_search_locations=[_pkg]
)
_mod = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _mod
_spec.loader.exec_module(_mod)
