"""Import path of the reference package (zhanglei1172/triton_int) served by ``triton_int_amd``.

Code written against the reference imports ``triton_int.nn.linear``, ``triton_int.nn.bmm``,
``triton_int.nn.fused``, ``triton_int.kernels.*`` and ``triton_int.functional.*``
(triton_int/nn/linear.py:18, triton_int/nn/bmm.py:10, triton_int/functional/bmm.py:6).  This package
holds no code of its own: every such name is bound to the ``triton_int_amd`` module of the same
relative path, so ``triton_int.nn.linear.W8A8B8O8Linear is triton_int_amd.nn.linear.W8A8B8O8Linear``.
"""
import importlib
import sys

import triton_int_amd as _impl

__version__ = _impl.__version__

# relative module paths of the reference tree that the int8 path covers (packages before their members)
ALIASES = (
    "nn", "nn.linear", "nn.bmm", "nn.fused",
    "functional", "functional.bmm", "functional.fused", "functional.quantization",
    "kernels", "kernels.linear", "kernels.bmm", "kernels.fused",
)

for _name in ALIASES:
    _mod = importlib.import_module("triton_int_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod
del _name, _mod
