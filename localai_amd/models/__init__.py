"""Model families.  `model_class(arch)` maps a checkpoint's architecture name (GGUF
general.architecture, or the name hf_checkpoint.open_model derives from config.json) to the class
LLMEngine builds; architectures not listed are the decoder-only transformer families of
decoder.DecoderModel."""
from __future__ import annotations

import importlib

# architecture -> (module, class); imported lazily: some families pull in optional dependencies
MODEL_CLASSES = {"suganex": ("localai_amd.models.suganex", "SuganexModel"),
                 "dadizen": ("localai_amd.models.dadizen", "DadizenModel"),
                 "vinozen": ("localai_amd.models.vinozen", "VinozenModel"),
                 "gosuvik": ("localai_amd.models.gosuvik", "GosuvikModel")}


def model_class(arch: str):
    mod, name = MODEL_CLASSES.get(arch, ("localai_amd.models.decoder", "DecoderModel"))
    return getattr(importlib.import_module(mod), name)
