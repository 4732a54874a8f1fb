"""MI355X-native 1-D neighbourhood attention (NA1D).

``nattn``  - drop-in for the reference's ``na1d_tensorcore.nattn`` entry points
``fused``  - the fused forward/backward operator
``_lib``   - ctypes binding of the C-ABI library ``libna1d.so``
"""
from .nattn import getNA1dFunction  # noqa: F401
from .fused import na1d_fused, na1d_fused_qkv  # noqa: F401
