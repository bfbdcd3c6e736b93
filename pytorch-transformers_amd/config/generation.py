"""Options of a generation call, with the reference's names, defaults and checks.

src/transformers/generation/configuration_utils.py:391-507 (fields and
defaults), :523-583 (mode from ``do_sample``), :585-838 (validate),
:1261-1302 (defaults taken from the model configuration), :1304-1327 (update).
Only the options of single-sequence greedy search and multinomial sampling are
built; ``seed`` is an addition (the reference samples from torch's global
generator, src/transformers/generation/utils.py:3277).  An option of the reference
that would change the tokens and is not built (``NOT_BUILT``) is refused by name when it
is set, wherever it comes from (a ``generation_config.json``, a keyword of
``generate``); options that change nothing here are kept in ``extra``.
"""
from __future__ import annotations

import dataclasses
import json
import os
import warnings
from typing import Any, Dict, List, Optional, Union

GENERATION_CONFIG_NAME = "generation_config.json"  # src/transformers/utils/__init__.py:268

# Options of the reference (configuration_utils.py:391-507) that change what is generated or returned and are not
# built, each with the values that leave it switched off
NOT_BUILT = {
    "num_beam_groups": (1, None), "penalty_alpha": (None,), "dola_layers": (None,), "diversity_penalty": (0.0, 0, None),
    "encoder_repetition_penalty": (1.0, 1, None), "force_words_ids": (None,), "constraints": (None,),
    "forced_bos_token_id": (None,), "forced_decoder_ids": (None,), "token_healing": (False, None),
    "guidance_scale": (None, 1.0, 1), "watermarking_config": (None,), "encoder_no_repeat_ngram_size": (0, None),
    "prompt_lookup_num_tokens": (None,), "assistant_early_exit": (None,), "output_attentions": (False, None),
    "output_hidden_states": (False, None),
}


def refuse_not_built(options: Dict[str, Any], source: str = "") -> None:
    """Raise for every option of ``options`` that is set and not built, naming them and where they came from."""
    asked = sorted(k for k, v in options.items() if k in NOT_BUILT and v not in NOT_BUILT[k])
    if options.get("num_beams") not in (None, 1):
        asked.append("num_beams")
    if asked:
        where = f" in {source}" if source else ""
        raise ValueError(
            f"generation option(s) set{where} that this engine has not built: "
            + ", ".join(f"{k}={options[k]!r}" for k in asked)
            + "; built are greedy search and sampling of one sequence per prompt with the processors of GenerationConfig")


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
    sequence_bias: Optional[Union[List[List[Any]], Dict[Any, float]]] = None
    forced_eos_token_id: Optional[Union[int, List[int]]] = None
    exponential_decay_length_penalty: Optional[List[Any]] = None
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
    #: options of the reference that change nothing here (beam-only settings, version stamps ...), kept as read
    extra: Dict[str, Any] = dataclasses.field(default_factory=dict)

    def __post_init__(self):
        if isinstance(self.sequence_bias, dict):  # the older form {tuple of ids: bias} (logits_process.py:1216-1220)
            if any(not isinstance(k, tuple) for k in self.sequence_bias):
                raise ValueError(f"`sequence_bias` has to be a dict with tuples as keys, but is {self.sequence_bias}.")
            self.sequence_bias = [[list(k), v] for k, v in self.sequence_bias.items()]
        if isinstance(self.exponential_decay_length_penalty, tuple):
            self.exponential_decay_length_penalty = list(self.exponential_decay_length_penalty)
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
        sb = self.sequence_bias
        if sb is not None:  # logits_process.py:1172-1214
            if not isinstance(sb, list) or len(sb) == 0:
                raise ValueError(f"`sequence_bias` has to be a non-empty dictionary, or non-empty list of lists but is {sb}.")
            ok = lambda e: (isinstance(e, (list, tuple)) and len(e) == 2 and isinstance(e[0], (list, tuple)) and len(e[0]) > 0
                            and all(isinstance(t, int) and not isinstance(t, bool) and t > 0 for t in e[0])
                            and isinstance(e[1], float))
            if any(not ok(e) for e in sb):
                raise ValueError("Each element in `sequence_bias` has to be a non-empty list of lists of positive integers "
                                 f"and float, but is {sb}.")
        fe = self.forced_eos_token_id
        if fe is not None:  # logits_process.py:1584-1585
            ids = [fe] if isinstance(fe, int) else fe
            if not isinstance(ids, list) or not ids or any(not isinstance(t, int) or isinstance(t, bool) or t < 0 for t in ids):
                raise ValueError(f"`eos_token_id` has to be a list of positive integers, but is {fe}")
        ed = self.exponential_decay_length_penalty
        if ed is not None:  # (start_index, decay_factor), configuration_utils.py:267-270
            if (not isinstance(ed, list) or len(ed) != 2 or not isinstance(ed[0], int) or isinstance(ed[0], bool)
                    or not isinstance(ed[1], (int, float)) or not (ed[1] > 0)):
                raise ValueError("`exponential_decay_length_penalty` has to be (start_index, decay_factor), an integer and "
                                 f"a positive number, but is {ed}")

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

    @property
    def forced_eos_token_ids(self) -> List[int]:
        f = self.forced_eos_token_id
        return [] if f is None else [int(f)] if isinstance(f, int) else [int(x) for x in f]

    def to_dict(self) -> Dict[str, Any]:
        d = dataclasses.asdict(self)
        d.update(d.pop("extra"))
        return d

    @classmethod
    def from_dict(cls, d: Dict[str, Any], source: str = "") -> "GenerationConfig":
        """From the contents of a ``generation_config.json``: the options built here become fields, an option that
        is set and not built raises by name (``source`` says where it stood), everything else is kept in ``extra``
        (the reference keeps unknown keys as attributes, configuration_utils.py:497-504)."""
        refuse_not_built(d, source)
        names = {f.name for f in dataclasses.fields(cls)} - {"extra"}
        extra = {k: v for k, v in d.items() if k not in names}
        try:
            return cls(**{k: v for k, v in d.items() if k in names}, extra=extra)
        except ValueError as e:
            if not source:
                raise
            raise ValueError(f"{source}: {e}") from None

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
                return cls.from_dict(json.load(f), source=path)
        if model_config is not None:
            return cls.from_model_config(model_config)
        return cls()

    def updated(self, **kwargs) -> "GenerationConfig":
        """A copy with ``kwargs`` set; unknown names raise (src/transformers/generation/utils.py:1543-1545)."""
        refuse_not_built(kwargs, "the arguments of generate()")
        names = {f.name for f in dataclasses.fields(self)} - {"extra"}
        unknown = sorted(set(kwargs) - names)
        if unknown:
            raise ValueError(f"unknown generation option(s): {', '.join(unknown)}")
        return dataclasses.replace(self, **kwargs)
