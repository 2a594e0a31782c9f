"""Import name of the engine.

The sources live in the sibling folder ``qwen-inference-lab_amd`` (a name Python
cannot import because of its hyphens); this package only points its search path
there and runs that folder's ``__init__``.
"""
from pathlib import Path as _Path

_SOURCE = _Path(__file__).resolve().parent.parent / 'qwen-inference-lab_amd'
__path__.append(str(_SOURCE))
exec(compile((_SOURCE / '__init__.py').read_text(), str(_SOURCE / '__init__.py'), 'exec'))
