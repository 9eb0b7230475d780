"""Import alias for the package directory `triton-snn-fusion_amd/`.

A hyphen cannot appear in a Python module name, so this module binds the directory as the package
`triton_snn_fusion_amd`: `import triton_snn_fusion_amd.runtime.snn_custom_ops` resolves inside `triton-snn-fusion_amd/`.
"""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "triton-snn-fusion_amd")]
__package__ = __name__

with open(_os.path.join(__path__[0], "__init__.py"), "r", encoding="utf-8") as _fh:
    exec(compile(_fh.read(), _os.path.join(__path__[0], "__init__.py"), "exec"), globals())
del _fh
