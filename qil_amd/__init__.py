"""Import name of the engine in a checkout that is not installed.

The sources live in the sibling folder ``qwen-inference-lab_amd`` (a name Python cannot import because
of its hyphens).  An installed package maps that folder to ``qil_amd`` itself (pyproject.toml); here the
same package is loaded from the folder under this name and takes this module's place.
"""
import importlib.util
import sys
from pathlib import Path

_source = Path(__file__).resolve().parent.parent / 'qwen-inference-lab_amd'
_spec = importlib.util.spec_from_file_location(__name__, _source / '__init__.py',
                                               submodule_search_locations=[str(_source)])
_package = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _package
_spec.loader.exec_module(_package)
