"""MPK (persistent kernel) front end."""
from .persistent_kernel import PersistentKernel
from .mpk import MPK, MPKMetadata
from .models import MirageModelConfig
from . import speculative
from .speculative import spec_decode_class

__all__ = ["MPK", "MPKMetadata", "spec_decode_class", "PersistentKernel", "MirageModelConfig", "speculative"]
