"""``qAB_v3`` of the reference's flash_recontruction/qAB_no_pe/v2.py:72-130: same contract as
``qAB`` in v1 and bound to the same HIP kernels (there is one implementation, not two)."""
from .v1 import qAB as qAB_v3  # noqa: F401
from .v1 import qAB  # noqa: F401
