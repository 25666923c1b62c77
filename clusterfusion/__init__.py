"""Drop-in name of the reference package: `import clusterfusion` resolves to the MI355X
implementation (reference clusterfusion/__init__.py:6-16 does the same re-export of its CUDA module)."""
from clusterfusionplus_amd import *  # noqa: F401,F403
from clusterfusionplus_amd import __all__  # noqa: F401
