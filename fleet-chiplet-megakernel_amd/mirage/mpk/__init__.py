"""MPK (persistent kernel) front end."""
from .persistent_kernel import PersistentKernel
from .mpk import MPK, MPKMetadata
from .models import MirageModelConfig


def spec_decode_class(method, **kwargs):
    """Speculative decoding is outside the decode megakernel's scope; only `None` is accepted
    (reference: python/mirage/mpk/speculative.py)."""
    if method is None:
        return None
    raise NotImplementedError(f"speculative decoding method '{method}' is not supported by the MI355X megakernel")
