"""Model registry: which class serves which architecture.

Built-in presets (random-init benchmark shapes) are looked up by name; a
checkpoint folder is dispatched on the `architecture` field of its
config.json."""
from __future__ import annotations

import json
import os
from typing import Callable, Dict

from kukeon_amd.engine.config import MODEL_PRESETS


def _llama(cfg, device, **kw):
    from kukeon_amd.models.llama import LlamaModel
    return LlamaModel(cfg, device=device)


def _mixtral(cfg, device, **kw):
    from kukeon_amd.models.mixtral import MixtralModel
    return MixtralModel(cfg, device=device)


def _lipedra(cfg, device, **kw):
    from kukeon_amd.models.lipedra import LipedraModel
    return LipedraModel(cfg, device=device, **kw)


def _rasesun(cfg, device, **kw):
    from kukeon_amd.models.rasesun import RasesunModel
    return RasesunModel(cfg, device=device, **kw)


def _dumovik(cfg, device, **kw):
    from kukeon_amd.models.dumovik import DumovikModel
    return DumovikModel(cfg, device=device, **kw)


def _bezizen(cfg, device, **kw):
    from kukeon_amd.models.bezizen import BezizenModel
    return BezizenModel(cfg, device=device, **kw)


# family -> constructor(cfg, device, **kw)
FAMILIES: Dict[str, Callable] = {
    "bezizen": _bezizen,
    "dumovik": _dumovik,
    "llama": _llama,
    "mixtral": _mixtral,
    "lipedra": _lipedra,
    "rasesun": _rasesun,
}

# config.json "architecture" -> family
ARCHITECTURES: Dict[str, str] = {
    "Lipedra": "lipedra",
    "Rasesun": "rasesun",
    "Dumovik": "dumovik",
    "Bezizen": "bezizen",
}


# family -> kernel groups its forward pass needs on a GPU (the sampler and
# the weight-streaming GEMMs of the "core" group are optional for these)
OP_GROUPS: Dict[str, tuple] = {
    "llama": ("core",),
    "mixtral": ("core",),
    "lipedra": ("mix",),
    "rasesun": ("recur",),
    "dumovik": ("hyb",),
    "bezizen": ("strm",),
}


def family_of(cfg) -> str:
    fam = getattr(cfg, "family", None)
    if fam:
        return fam
    return "mixtral" if getattr(cfg, "is_moe", False) else "llama"


def build_model(cfg, device, **kw):
    """Instantiate (random-init) the model class that serves `cfg`."""
    return FAMILIES[family_of(cfg)](cfg, device, **kw)


def _lipedra_preset(**kw):
    def make():
        from kukeon_amd.models.lipedra import lipedra_bench
        return lipedra_bench(**kw)
    return make


# random-weight Lipedra stacks at Llama-3-8B layer sizes: 32 layers, every
# second layer reading its predecessor's cache; and a small one for tests
LIPEDRA_PRESETS = {
    "lipedra-8b-like": _lipedra_preset(width=4096, layers=32, heads=32,
                                       kv_heads=8, dim=64, vdim=128,
                                       ff=14336, vocab=128256, share_every=2,
                                       name="lipedra-8b-like"),
    "tiny-lipedra": _lipedra_preset(width=192, layers=3, heads=6, kv_heads=2,
                                    dim=16, vdim=32, ff=320, vocab=384,
                                    share_every=3, name="tiny-lipedra"),
}


def _rasesun_preset(**kw):
    def make():
        from kukeon_amd.models.rasesun import rasesun_bench
        return rasesun_bench(**kw)
    return make


# random-weight Rasesun stacks: three state-space layers to one latent
# attention layer at Llama-3-8B width, and a small one for tests
RASESUN_PRESETS = {
    "rasesun-8b-like": _rasesun_preset(width=4096, layers=32, heads=32,
                                       ff=14336, vocab=128256,
                                       name="rasesun-8b-like"),
    "tiny-rasesun": _rasesun_preset(width=128, layers=4, heads=2, ff=256,
                                    vocab=384, window=24, experts=4,
                                    name="tiny-rasesun"),
}


def _dumovik_preset(**kw):
    def make():
        from kukeon_amd.models.dumovik import dumovik_bench
        return dumovik_bench(**kw)
    return make


# random-weight Dumovik stacks: periods of chunked attention, two linear
# attention layers and latent attention at Llama-3-8B width, and a small one
DUMOVIK_PRESETS = {
    "dumovik-8b-like": _dumovik_preset(width=4096, layers=32, heads=32,
                                       kv_heads=8, ff=14336, vocab=128256,
                                       name="dumovik-8b-like"),
    "tiny-dumovik": _dumovik_preset(width=128, layers=8, heads=2, kv_heads=1,
                                    ff=256, vocab=384, chunk=24, experts=4,
                                    name="tiny-dumovik"),
}


def _bezizen_preset(**kw):
    def make():
        from kukeon_amd.models.bezizen import bezizen_bench
        return bezizen_bench(**kw)
    return make


# random-weight Bezizen stacks: three wkv layers to one parallel layer over
# four residual streams at Llama-3-8B width, and a small one
BEZIZEN_PRESETS = {
    "bezizen-8b-like": _bezizen_preset(width=4096, layers=32, heads=32,
                                       kv_heads=8, ff=14336, vocab=128256,
                                       name="bezizen-8b-like"),
    "tiny-bezizen": _bezizen_preset(width=128, layers=4, heads=4, kv_heads=2,
                                    ff=256, vocab=384, window=24, experts=8,
                                    streams=2, max_positions=512,
                                    name="tiny-bezizen"),
}


def preset_names():
    return sorted(list(MODEL_PRESETS) + list(LIPEDRA_PRESETS) +
                  list(RASESUN_PRESETS) + list(DUMOVIK_PRESETS) +
                  list(BEZIZEN_PRESETS))


def preset(name: str):
    if name in BEZIZEN_PRESETS:
        return BEZIZEN_PRESETS[name]()
    if name in DUMOVIK_PRESETS:
        return DUMOVIK_PRESETS[name]()
    if name in LIPEDRA_PRESETS:
        return LIPEDRA_PRESETS[name]()
    if name in RASESUN_PRESETS:
        return RASESUN_PRESETS[name]()
    if name not in MODEL_PRESETS:
        raise KeyError(f"unknown model preset {name!r}; known: "
                       f"{preset_names()}")
    return MODEL_PRESETS[name]()


def load_checkpoint(model_dir: str, device, dtype: str = "bf16"):
    """-> (cfg, model) for a folder with config.json + model.safetensors."""
    with open(os.path.join(model_dir, "config.json")) as f:
        arch = json.load(f).get("architecture")
    fam = ARCHITECTURES.get(arch)
    if fam is None:
        raise ValueError(f"no model class registered for architecture "
                         f"{arch!r}; known: {sorted(ARCHITECTURES)}")
    if fam == "lipedra":
        from kukeon_amd.models.lipedra import LipedraModel
        return LipedraModel.from_checkpoint(model_dir, device=device,
                                            dtype=dtype)
    if fam == "rasesun":
        from kukeon_amd.models.rasesun import RasesunModel
        return RasesunModel.from_checkpoint(model_dir, device=device,
                                            dtype=dtype)
    if fam == "dumovik":
        from kukeon_amd.models.dumovik import DumovikModel
        return DumovikModel.from_checkpoint(model_dir, device=device,
                                            dtype=dtype)
    if fam == "bezizen":
        from kukeon_amd.models.bezizen import BezizenModel
        return BezizenModel.from_checkpoint(model_dir, device=device,
                                            dtype=dtype)
    raise ValueError(f"family {fam} has no checkpoint loader")
