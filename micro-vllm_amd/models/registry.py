"""Which model family a checkpoint's config.json names, and how each family is loaded and run.

A family = (configuration reader, model object, runner and cache manager the engine builds for it):
  "llama"  - the Llama-shaped stacks (Qwen-1, Llama, Mistral, Qwen2 naming), padded prefill and
             graph-captured single-token decode over one KV geometry (ModelPrefillRunner /
             ModelGraphRunner / KVCacheManager);
  "ragged" - stacks with an fp32 residual stream whose layers are listed one by one (recurrent
             mixers, windowed or latent attention, dense or routed feed-forwards), run step by step
             over ragged batches (RaggedRunner / HybridCacheManager): Pagazen, Fagunex, Nesisun, Solopel.
"""
from typing import Callable, Dict

_ARCHITECTURES: Dict[str, Callable] = {}


def register(architecture: str, loader: Callable):
    """loader(config_json: dict, files, name: str) -> model object with `.config` and `.family`."""
    _ARCHITECTURES[architecture] = loader


def _load_pagazen(config_json, files, name):
    from .pagazen import PagazenConfig, PagazenModel, tensor_shapes
    cfg = PagazenConfig.from_json(config_json, name)
    for tensor, shape in tensor_shapes(cfg).items():
        if tensor not in files:
            raise KeyError(f"tensor {tensor!r} {shape} is not in the checkpoint")
    return PagazenModel(cfg, files)


def _load_fagunex(config_json, files, name):
    from .fagunex import FagunexConfig, FagunexModel, tensor_shapes
    cfg = FagunexConfig.from_json(config_json, name)
    for tensor, shape in tensor_shapes(cfg).items():
        if tensor not in files:
            raise KeyError(f"tensor {tensor!r} {shape} is not in the checkpoint")
    return FagunexModel(cfg, files)


def _load_nesisun(config_json, files, name):
    from .nesisun import NesisunConfig, NesisunModel, tensor_shapes
    cfg = NesisunConfig.from_json(config_json, name)
    for tensor, shape in tensor_shapes(cfg).items():
        if tensor not in files:
            raise KeyError(f"tensor {tensor!r} {shape} is not in the checkpoint")
    return NesisunModel(cfg, files)


def _load_solopel(config_json, files, name):
    from .solopel import SolopelConfig, SolopelModel, tensor_shapes
    cfg = SolopelConfig.from_json(config_json, name)
    for tensor, shape in tensor_shapes(cfg).items():
        if tensor not in files:
            raise KeyError(f"tensor {tensor!r} {shape} is not in the checkpoint")
    return SolopelModel(cfg, files)


register("Pagazen", _load_pagazen)
register("Fagunex", _load_fagunex)
register("Nesisun", _load_nesisun)
register("Solopel", _load_solopel)


def loader_for(config_json: dict):
    """The registered loader for config.json's `architecture`, or None (Llama-shaped checkpoints
    carry `model_type` instead and go the tensor-name way of core/model_loader.py)."""
    return _ARCHITECTURES.get(config_json.get("architecture"))


def family_of(model) -> str:
    return getattr(model, "family", "llama")
