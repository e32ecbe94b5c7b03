"""The Python entry point.

Shaped after the reference's C surface (/root/reference/capi/include/sonicboom/capi.h:600-829):
a model is loaded once (``boom_llm_model_load``), sessions are made from it
(``boom_llm_session_new``) and own the cache, a session runs steps and
generation (``boom_llm_prefill`` / ``boom_llm_decode``) with the sampling
options of ``boom_llm_sampling`` under the same names, and the model's own stop
tokens are readable (``boom_llm_model_eos``).  Tokens in, tokens out: there is
no tokenizer here.

    model = Model.load("/path/to/folder", dtype="bfloat16")
    session = model.session(max_tokens=8192)
    outs = session.generate([[1, 2, 3], [4, 5]], temperature=0.8, seed=7, max_tokens=32)
"""
from __future__ import annotations

from typing import Callable, Iterable, List, Optional, Sequence

from .engine import DecoderModel, Engine, StepEntry, generate
from .engine.prefix import KeptSequences
from .sampling import SamplingParams


class Model:
    def __init__(self, decoder: DecoderModel):
        self.decoder = decoder

    @classmethod
    def load(cls, folder: str, dtype: str = "bfloat16", device=None, fast_kernels: bool = True) -> "Model":
        """Load config.json + safetensors; the model class is chosen by config.json's ``architectures``."""
        return cls(DecoderModel.from_folder(folder, dtype, device, fast_kernels))

    @classmethod
    def random(cls, config, seed: int = 0, dtype: str = "bfloat16", device=None,
               fast_kernels: bool = True) -> "Model":
        """A model of random weights for a configuration (typed, or a config.json dict)."""
        return cls(DecoderModel.from_random(config, seed, dtype, device, fast_kernels))

    @property
    def arch(self) -> str:
        return self.decoder.spec.architecture

    @property
    def eos(self) -> tuple:
        return tuple(self.decoder.spec.stop_tokens)

    @property
    def vocab_size(self) -> int:
        return self.decoder.vocab

    def session(self, max_tokens: int, max_slots: Optional[int] = None,
                max_positions: Optional[int] = None) -> "Session":
        """A cache for at most ``max_tokens`` live tokens (each sequence rounded up to 64).
        ``max_positions`` bounds a sequence's length: None takes the model's own maximum of
        positions, 0 sets no bound."""
        return Session(self, max_tokens, max_slots, max_positions)


class Session:
    def __init__(self, model: Model, max_tokens: int, max_slots: Optional[int] = None,
                 max_positions: Optional[int] = None):
        self.model = model
        self.engine = Engine(model.decoder, max_tokens, max_slots, max_positions=max_positions)
        self.kept = KeptSequences(self.engine)      # sequences the last generate(keep=True) left
        self.keep = False                           # what generate does when it is not told

    def alloc_slot(self) -> int:
        return self.engine.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.engine.free_slot(slot)

    def step(self, entries: Sequence):
        """entries: (slot, tokens, want) triples or StepEntry; float32 logits [wanted, vocab] on the device."""
        return self.engine.step([e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries])

    def generate(self, prompts: Sequence[Sequence[int]], temperature: float = 0.0, top_p: float = 1.0,
                 top_k: int = 0, seed: int = 0, max_tokens: int = 16, min_p: float = 0.0,
                 repeat_penalty: float = 1.0, repeat_last_n: int = 64, presence_penalty: float = 0.0,
                 frequency_penalty: float = 0.0, stop_tokens: Optional[Iterable[int]] = None,
                 max_batch: int = 64, callback: Optional[Callable] = None,
                 allowed: Optional[Callable] = None, keep: Optional[bool] = None) -> List[List[int]]:
        """``allowed(i, history)`` returns the bitmap of the ids request i may choose next (bit
        i & 7 of byte i >> 3 for id i; None: any): the mask of constrained decoding.

        ``keep`` (default: the session's ``keep`` attribute): the requests' sequences stay in
        the cache when they end, and a prompt of the next call that starts with the tokens of
        one of them feeds only the rest (prefix reuse: a conversation that goes on; at most all
        but the prompt's last token are reused).  ``reused`` then tells how many tokens of each
        prompt were not fed again.  The produced tokens do not depend on it.  A call without
        ``keep`` frees what an earlier one kept."""
        keep = self.keep if keep is None else bool(keep)
        params = SamplingParams(temperature=temperature, top_p=top_p, top_k=top_k, seed=seed,
                                max_tokens=max_tokens, min_p=min_p, repeat_penalty=repeat_penalty,
                                repeat_last_n=repeat_last_n, presence_penalty=presence_penalty,
                                frequency_penalty=frequency_penalty)
        if not keep:
            self.forget()
        return generate(self.engine, prompts, params, stop_tokens, max_batch, callback, allowed=allowed,
                        kept=self.kept if keep else None)

    @property
    def reused(self) -> List[int]:
        """Per prompt of the last ``generate(keep=True)``: the tokens taken from a kept sequence."""
        return list(self.kept.reused)

    def forget(self) -> None:
        """Free the sequences that ``generate(keep=True)`` has left in the cache."""
        self.kept.drop_all()
        self.kept.reused = []
