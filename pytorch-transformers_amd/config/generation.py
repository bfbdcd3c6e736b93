"""Options of a generation call, with the reference's names, defaults and checks.

src/transformers/generation/configuration_utils.py:391-507 (fields and
defaults), :523-583 (mode from ``do_sample``), :585-838 (validate),
:1261-1302 (defaults taken from the model configuration), :1304-1327 (update).
Only the options of single-sequence greedy search and multinomial sampling are
kept; ``seed`` is an addition (the reference samples from torch's global
generator, src/transformers/generation/utils.py:3277).
"""
from __future__ import annotations

import dataclasses
import json
import os
import warnings
from typing import Any, Dict, List, Optional, Union

GENERATION_CONFIG_NAME = "generation_config.json"  # src/transformers/utils/__init__.py:268


@dataclasses.dataclass
class GenerationConfig:
    # length
    max_length: int = 20
    max_new_tokens: Optional[int] = None
    min_length: int = 0
    min_new_tokens: Optional[int] = None
    max_time: Optional[float] = None
    stop_strings: Optional[Union[str, List[str]]] = None
    # strategy
    do_sample: bool = False
    num_beams: int = 1
    # cache
    use_cache: bool = True
    cache_implementation: Optional[str] = None
    # logits
    temperature: Optional[float] = 1.0
    top_k: Optional[int] = 50
    top_p: Optional[float] = 1.0
    min_p: Optional[float] = None
    typical_p: Optional[float] = 1.0
    epsilon_cutoff: Optional[float] = 0.0
    eta_cutoff: Optional[float] = 0.0
    repetition_penalty: Optional[float] = 1.0
    no_repeat_ngram_size: Optional[int] = 0
    bad_words_ids: Optional[List[List[int]]] = None
    suppress_tokens: Optional[List[int]] = None
    begin_suppress_tokens: Optional[List[int]] = None
    renormalize_logits: bool = False
    remove_invalid_values: bool = False
    # outputs
    num_return_sequences: int = 1
    output_scores: bool = False
    output_logits: Optional[bool] = None
    return_dict_in_generate: bool = False
    # special tokens
    pad_token_id: Optional[int] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[Union[int, List[int]]] = None
    # sampling seed (ours)
    seed: int = 0

    def __post_init__(self):
        self.validate()

    # ------------------------------------------------------------------
    def validate(self) -> None:
        """configuration_utils.py:585-838, for the options kept here."""
        if self.num_beams != 1:
            raise ValueError("beam search is not built: num_beams must be 1")
        if self.cache_implementation not in (None, "paged"):
            raise ValueError(
                f"cache_implementation={self.cache_implementation!r} is not built; the engine has one cache "
                "(pages of a pool, a slot per sequence): use None")
        if not self.use_cache:
            raise ValueError("use_cache=False is not built: the step function always runs from the cache")
        if self.max_new_tokens is not None and self.max_new_tokens <= 0:  # :599-600
            raise ValueError(f"`max_new_tokens` must be greater than 0, but is {self.max_new_tokens}.")
        if self.max_length is not None and self.max_length <= 0:
            raise ValueError(f"`max_length` must be greater than 0, but is {self.max_length}.")
        if self.min_length is not None and self.min_length < 0:
            raise ValueError(f"`min_length` has to be a non-negative integer, but is {self.min_length}")
        if self.min_new_tokens is not None and self.min_new_tokens < 0:
            raise ValueError(f"`min_new_tokens` has to be a non-negative integer, but is {self.min_new_tokens}")
        if self.num_return_sequences < 1:
            raise ValueError("`num_return_sequences` has to be at least 1")
        if not self.do_sample:
            # :609-653: sampling-only flags set while sampling is off only warn in the reference
            if self.num_return_sequences != 1:  # :706-711
                raise ValueError(
                    "Greedy methods without beam search do not support `num_return_sequences` different than 1 "
                    f"(got {self.num_return_sequences}).")
            for name, default in (("temperature", 1.0), ("top_p", 1.0), ("min_p", None), ("typical_p", 1.0),
                                  ("epsilon_cutoff", 0.0), ("eta_cutoff", 0.0)):
                v = getattr(self, name)
                if v is not None and v != default:
                    warnings.warn(
                        f"`do_sample` is set to `False`. However, `{name}` is set to `{v}` -- this flag is only used "
                        "in sample-based generation modes.", UserWarning, stacklevel=3)
        else:
            # the processors' own checks (src/transformers/generation/logits_process.py)
            t = self.temperature
            if t is not None and (not isinstance(t, float) or not (t > 0)):  # :274-283
                msg = (f"`temperature` (={t}) has to be a strictly positive float, otherwise your next token "
                       "scores will be invalid.")
                if isinstance(t, float) and t == 0.0:
                    msg += " If you're looking for greedy decoding strategies, set `do_sample=False`."
                raise ValueError(msg)
            if self.top_k is not None and self.top_k != 0:
                if not isinstance(self.top_k, int) or self.top_k < 0:  # :505-507
                    raise ValueError(f"`top_k` has to be a strictly positive integer, but is {self.top_k}")
            if self.top_p is not None and (self.top_p < 0 or self.top_p > 1.0):  # :441-444
                raise ValueError(f"`top_p` has to be a float > 0 and < 1, but is {self.top_p}")
            if self.min_p is not None and not (0 <= self.min_p <= 1.0):  # :568-570
                raise ValueError(f"`min_p` has to be a float in the [0, 1] interval, but is {self.min_p}")
            if self.typical_p is not None and self.typical_p < 1.0 and not (self.typical_p > 0):  # :651-653
                raise ValueError(f"`typical_p` has to be a float > 0 and < 1, but is {self.typical_p}")
        n = self.no_repeat_ngram_size
        if n is not None and n != 0 and (not isinstance(n, int) or n < 0):  # logits_process.py:949-951
            raise ValueError(f"`ngram_size` has to be a strictly positive integer, but is {n}")
        bw = self.bad_words_ids
        if bw is not None:  # logits_process.py:1288-1299
            if not isinstance(bw, list) or len(bw) == 0:
                raise ValueError(f"`bad_words_ids` has to be a non-empty list, but is {bw}.")
            if any(not isinstance(w, list) for w in bw):
                raise ValueError(f"`bad_words_ids` has to be a list of lists, but is {bw}.")
            if any(len(w) == 0 or any((not isinstance(t, int) or t < 0) for t in w) for w in bw):
                raise ValueError(f"Each list in `bad_words_ids` has to be a list of positive integers, but is {bw}.")
        rp = self.repetition_penalty
        if rp is not None and (not isinstance(rp, float) or not (rp > 0)):  # :329-331
            raise ValueError(f"`penalty` has to be a strictly positive float, but is {rp}")

    # ------------------------------------------------------------------
    @property
    def eos_token_ids(self) -> List[int]:
        """``eos_token_id`` may be an int or a list (src/transformers/generation/utils.py:1859-1861)."""
        e = self.eos_token_id
        if e is None:
            return []
        if isinstance(e, int):
            return [e]
        return [int(x) for x in e]

    def to_dict(self) -> Dict[str, Any]:
        return dataclasses.asdict(self)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GenerationConfig":
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in names})

    @classmethod
    def from_model_config(cls, model_config) -> "GenerationConfig":
        """Special token ids come from the model configuration (:1261-1302)."""
        d = {k: v for k, v in model_config.to_dict().items() if v is not None}
        keep = {k: d[k] for k in ("pad_token_id", "bos_token_id", "eos_token_id") if k in d}
        return cls(**keep)

    @classmethod
    def from_pretrained(cls, folder: str, model_config=None) -> "GenerationConfig":
        """generation_config.json if the folder has one, else from the model configuration."""
        path = os.path.join(folder, GENERATION_CONFIG_NAME)
        if os.path.isfile(path):
            with open(path, "r", encoding="utf-8") as f:
                return cls.from_dict(json.load(f))
        if model_config is not None:
            return cls.from_model_config(model_config)
        return cls()

    def updated(self, **kwargs) -> "GenerationConfig":
        """A copy with ``kwargs`` set; unknown names raise (src/transformers/generation/utils.py:1543-1545)."""
        names = {f.name for f in dataclasses.fields(self)}
        unknown = sorted(set(kwargs) - names)
        if unknown:
            raise ValueError(f"unknown generation option(s): {', '.join(unknown)}")
        return dataclasses.replace(self, **kwargs)
