"""Import name of the engine.

The sources live in the folder ``distributed-llm-inference_amd`` at the repository root; a hyphen
cannot appear in a Python module name, so this package points its search path there. Every
sub-package (``dli_amd.config``, ``dli_amd.parts``, ...) is found in that folder.
"""

from pathlib import Path as _Path

SOURCE_ROOT = _Path(__file__).resolve().parent.parent / "distributed-llm-inference_amd"
__path__.append(str(SOURCE_ROOT))

__version__ = "0.1.0"
