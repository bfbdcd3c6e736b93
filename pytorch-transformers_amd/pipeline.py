"""``pipeline("text-generation", model=folder)``: the Python entry point in the reference's manner.

The reference's pipeline tokenizes, calls ``generate`` and decodes
(src/transformers/pipelines/text_generation.py:39-449; ``_forward`` :349-389), returning for every
input a list of ``{"generated_text": ...}`` (or ``{"generated_token_ids": ...}`` with
``return_tensors=True``, :391-449).  The engine starts at token ids: a prompt may be a list of ids,
and text is accepted when the model folder has a ``tokenizer.json`` that the ``tokenizers`` package
can read (a text <-> ids utility only; no model code of any package is used).
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence, Union

from .auto import AutoModelForCausalLM

Prompt = Union[str, Sequence[int]]


def load_tokenizer(folder: str):
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(path)


class TextGenerationPipeline:
    def __init__(self, model, tokenizer=None):
        self.model = model
        self.tokenizer = tokenizer

    def _encode(self, prompt: Prompt, prefix: str = "") -> List[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("text prompts need a tokenizer.json in the model folder; pass token ids instead")
            return list(self.tokenizer.encode(prefix + prompt).ids)
        return [int(t) for t in prompt]

    def __call__(self, prompts: Union[Prompt, Sequence[Prompt]], *, return_tensors: Optional[bool] = None,
                 return_full_text: bool = True, prefix: str = "", batch_size: Optional[int] = None,
                 **generate_kwargs):
        single = isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], int))
        items = [prompts] if single else list(prompts)
        ids = [self._encode(p, prefix) for p in items]
        n_ret = int(generate_kwargs.get("num_return_sequences", 1))
        seqs = self.model.generate(ids, batch_size=batch_size, tokenizer=self.tokenizer, **generate_kwargs)
        as_text = self.tokenizer is not None and not return_tensors and all(isinstance(p, str) for p in items)
        out = []
        for i, p in enumerate(ids):
            records = []
            for seq in seqs[i * n_ret:(i + 1) * n_ret]:
                toks = seq if return_full_text else seq[len(p):]
                if as_text:
                    records.append({"generated_text": self.tokenizer.decode(toks)})
                else:
                    records.append({"generated_token_ids": toks})
            out.append(records)
        return out[0] if single else out


def pipeline(task: str = "text-generation", model: Optional[str] = None, dtype="bfloat16", device="cuda:0",
             tokenizer=None, tuning_table=None, **kwargs) -> TextGenerationPipeline:
    """``tuning_table``: timed choices between kernels for the model to take (``CausalLM.tune``'s result, or the
    path of a JSON file that holds it)."""
    if task != "text-generation":
        raise ValueError(f"task {task!r} is not built; only 'text-generation'")
    if model is None:
        raise ValueError("pipeline needs model=<folder with config.json and model.safetensors>")
    if isinstance(model, str):
        tokenizer = tokenizer or load_tokenizer(model)
        model = AutoModelForCausalLM.from_pretrained(model, dtype=kwargs.pop("torch_dtype", None) or dtype, device=device,
                                                     tuning_table=tuning_table)
    elif tuning_table is not None:
        model.tune(table=tuning_table)
    return TextGenerationPipeline(model, tokenizer)
