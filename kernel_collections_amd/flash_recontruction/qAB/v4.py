"""Same contract as ``qAB`` in v1 (the reference keeps several Triton variants of one function,
flash_recontruction/qAB/{ref,v3,v4}.py); here every name binds to the single HIP implementation."""
from .v1 import qAB  # noqa: F401
