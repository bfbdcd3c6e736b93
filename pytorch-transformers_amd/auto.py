"""``AutoModelForCausalLM``: from a model folder, or a configuration, to a model on the GPU.

The reference resolves ``config.json``'s ``model_type`` to a configuration class and that to a model
class (src/transformers/models/auto/auto_factory.py:419-590); here both come from one registry and
the model class is always ``engine.model.CausalLM``, built from the parts the registered builder
lists.
"""
from __future__ import annotations


class AutoModelForCausalLM:
    @staticmethod
    def from_pretrained(folder: str, dtype="bfloat16", device="cuda:0", strict: bool = True, torch_dtype=None,
                        tuning_table=None):
        from .engine.model import CausalLM

        return CausalLM.from_pretrained(folder, dtype=torch_dtype or dtype, device=device, strict=strict,
                                        tuning_table=tuning_table)

    @staticmethod
    def from_config(config, seed: int = 0, dtype="bfloat16", device="cuda:0", torch_dtype=None, **kwargs):
        from .engine.model import CausalLM

        return CausalLM.from_config(config, seed=seed, dtype=torch_dtype or dtype, device=device, **kwargs)
