"""Model registry: which configuration class and which decoder a checkpoint folder's config.json selects.

A folder holds config.json and model.safetensors.  The design is named by `architecture` (this repository's own designs)
or by `architectures` / `model_type` (Hugging Face names of the dense families).  `load_model_dir` reads the configuration,
`model_class(cfg)` gives the decoder the engine builds, `load_weights` fills it from the safetensors file.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Callable, Dict, Tuple

from .hybrid import HybridConfig, HybridDecoder, bedarax_config, givavik_config, piladra_config
from .model import DenseDecoder, ModelConfig


def dense_config_from_hf(cfg: Dict[str, Any]) -> ModelConfig:
    """config.json of a Qwen3 / Qwen2 / Llama checkpoint -> ModelConfig (the fields of P/models/config.py:19-87)."""
    heads = int(cfg["num_attention_heads"])
    kind = cfg.get("model_type", "")
    return ModelConfig(
        num_layers=int(cfg["num_hidden_layers"]), num_qo_heads=heads, num_kv_heads=int(cfg.get("num_key_value_heads", heads)),
        head_dim=int(cfg.get("head_dim") or cfg["hidden_size"] // heads), hidden_size=int(cfg["hidden_size"]),
        vocab_size=int(cfg["vocab_size"]), intermediate_size=int(cfg["intermediate_size"]),
        rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-6)), rope_base=float(cfg.get("rope_theta", 10000.0)),
        rope_scaling=cfg.get("rope_scaling"), max_position=int(cfg.get("max_position_embeddings", 4096)),
        tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)), qk_norm=kind == "qwen3", name=kind or "dense")


def _load_dense(model: DenseDecoder, state: Dict[str, Any]) -> None:
    model.load_hf_state(state)


def _load_hybrid(model: HybridDecoder, state: Dict[str, Any]) -> None:
    model.load_state(state)


# name in config.json -> (configuration reader, decoder class, weight loader)
ARCHITECTURES: Dict[str, Tuple[Callable[[Dict[str, Any]], Any], type, Callable[[Any, Dict[str, Any]], None]]] = {
    "Nidorax": (HybridConfig.from_json, HybridDecoder, _load_hybrid),
    "Bedarax": (bedarax_config, HybridDecoder, _load_hybrid),
    "Givavik": (givavik_config, HybridDecoder, _load_hybrid),
    "Piladra": (piladra_config, HybridDecoder, _load_hybrid),
    "Qwen3ForCausalLM": (dense_config_from_hf, DenseDecoder, _load_dense),
    "Qwen2ForCausalLM": (dense_config_from_hf, DenseDecoder, _load_dense),
    "LlamaForCausalLM": (dense_config_from_hf, DenseDecoder, _load_dense),
}


def architecture_of(cfg: Dict[str, Any]) -> str:
    names = [cfg["architecture"]] if "architecture" in cfg else list(cfg.get("architectures") or [])
    for n in names:
        if n in ARCHITECTURES:
            return n
    raise ValueError(f"no model registered for {names or 'a config.json without an architecture name'}; "
                     f"known: {sorted(ARCHITECTURES)}")


def model_class(cfg: Any) -> type:
    """The decoder class for a configuration object."""
    return HybridDecoder if isinstance(cfg, HybridConfig) else DenseDecoder


def checkpoint_shapes(path) -> Dict[str, Tuple[int, ...]]:
    """Tensor name -> shape from the header of the folder's model.safetensors (8-byte little-endian length, then that many
    bytes of JSON); {} when there is no such file.  No tensor data is read."""
    file = Path(path) / "model.safetensors"
    if not file.exists():
        return {}
    with open(file, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items() if k != "__metadata__"}


def load_model_dir(path) -> Tuple[Any, str]:
    """-> (configuration object, registered architecture name) of the folder's config.json.  A reader that declares a `shapes`
    parameter also gets the checkpoint's tensor shapes: some designs leave sizes to them."""
    import inspect

    with open(Path(path) / "config.json") as f:
        raw = json.load(f)
    name = architecture_of(raw)
    reader = ARCHITECTURES[name][0]
    if "shapes" in inspect.signature(reader).parameters:
        return reader(raw, shapes=checkpoint_shapes(path)), name
    return reader(raw), name


def load_weights(model: Any, path, name: str) -> None:
    """model.safetensors of the folder -> the decoder's tensors (host read, then one copy per tensor to the device)."""
    from safetensors.torch import load_file

    ARCHITECTURES[name][2](model, load_file(str(Path(path) / "model.safetensors")))
