"""Import name of the framework whose files lie in `gene-llm-inference-engine_amd/`.

That folder's name is not a Python identifier, so this module stands in for it as a package:
`import geneinfer_amd.config` finds `gene-llm-inference-engine_amd/config/`.
"""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "gene-llm-inference-engine_amd")]
_init = _os.path.join(__path__[0], "__init__.py")
with open(_init) as _f:
    exec(compile(_f.read(), _init, "exec"))
del _os, _init, _f
