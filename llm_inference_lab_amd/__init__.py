"""Importable name of the framework.

The sources live in the folder ``llm-inference-lab_amd/`` next to this one; a
hyphen cannot appear in a Python module name, so this package points its
search path there and runs that folder's ``__init__.py`` as its own.
"""
import pathlib as _pathlib

_src = _pathlib.Path(__file__).resolve().parent.parent / "llm-inference-lab_amd"
__path__ = [str(_src)]
exec(compile((_src / "__init__.py").read_text(), str(_src / "__init__.py"), "exec"))
