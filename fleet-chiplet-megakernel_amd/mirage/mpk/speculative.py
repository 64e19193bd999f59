"""Speculative-decoding configurations (reference: python/mirage/mpk/speculative.py).

Only prompt lookup has tasks behind it -- in the reference as here: a decoding request's guesses are the tokens that
followed the earliest earlier occurrence of its last `ngram_size` tokens (PersistentKernel.prompt_lookup_spec_handler),
checked against what the model samples by PersistentKernel.prompt_lookup_verify_handler.  `LookaheadConfig` exists as a
configuration class in the reference but no handler is registered for it (persistent_kernel.py:410-415)."""
from dataclasses import dataclass


@dataclass
class SpecDecodeConfig:
    method: str


@dataclass
class LookaheadConfig(SpecDecodeConfig):
    method: str = "lookahead"
    spec_length: int = 7


@dataclass
class PromptLookupConfig(SpecDecodeConfig):
    method: str = "promptlookup"
    ngram_size: int = 3
    spec_length: int = 5


def spec_decode_class(spec_decode, ngram_size: int = 3, spec_length: int = 5):
    if spec_decode is None:
        return None
    if spec_decode == "promptlookup":
        return PromptLookupConfig(ngram_size=ngram_size, spec_length=spec_length)
    if spec_decode == "lookahead":
        return LookaheadConfig(spec_length=spec_length)
    raise NotImplementedError(f"Spec decode method {spec_decode} not implemented")
