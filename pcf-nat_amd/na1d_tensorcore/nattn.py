"""Import shim: with ``pcf-nat_amd`` on ``sys.path`` the reference models'
``from na1d_tensorcore.nattn import getNA1dFunction``
(models/PCF_NATransformer.py:22, models/MFA_NATransformer.py:21) resolves to the
MI355X implementation without editing them."""
from na1d_amd.nattn import (  # noqa: F401
    bf16_ANA1d_AV_Function,
    bf16_ANA1d_QK_Function,
    fp16_ANA1d_AV_Function,
    fp16_ANA1d_QK_Function,
    getNA1dFunction,
)
