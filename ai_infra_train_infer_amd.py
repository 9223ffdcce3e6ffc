"""Import name for the package in `ai-infra-train-infer_amd/` (a hyphen cannot appear in an
import statement): `import ai_infra_train_infer_amd as pa` loads that directory as this module,
and `ai_infra_train_infer_amd.attention` etc. resolve inside it."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ai-infra-train-infer_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_mod = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _mod
_spec.loader.exec_module(_mod)
