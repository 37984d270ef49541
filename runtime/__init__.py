"""Import name of the engine.  The sources live in the folder
``cuda-inference-serving-runtime_amd`` beside this one, whose name is not a
Python identifier; this package points its search path there and runs that
folder's ``__init__.py`` as its own, so ``runtime.engine``, ``python -m
runtime`` and so on resolve to those files."""
from pathlib import Path as _Path

_src = _Path(__file__).resolve().parent.parent / "cuda-inference-serving-runtime_amd"
__path__ = [str(_src)]
exec(compile((_src / "__init__.py").read_text(), str(_src / "__init__.py"), "exec"))
