"""Model construction: presets (``configs``), random-init or checkpoint weights."""
from __future__ import annotations

from pathlib import Path
from typing import Optional

import torch

from ..parallel.tp import SINGLE, TPGroup
from .bert import EncoderModel
from .configs import (DECODERS, ENCODERS, DecoderConfig, EncoderConfig, FusasunConfig, LebepelConfig, LumedraConfig, PemidraConfig, decoder_config,
                      encoder_config)
from . import llama
from .fusasun import FusasunModel
from .lebepel import LebepelModel
from .llama import LlamaModel
from .lumedra import LumedraModel
from .opt import OPTModel
from .pemidra import PemidraModel, ranks_from_state_dict

# decoder architectures by ``cfg.arch``
DECODER_CLASSES = {"llama": LlamaModel, "opt": OPTModel, "lebepel": LebepelModel, "pemidra": PemidraModel,
                   "fusasun": FusasunModel, "lumedra": LumedraModel}
# designs with a checkpoint format of their own (config.json read by ``<Config>.from_json``, tensors by
# ``load_state_dict_native``)
NATIVE_CONFIGS = {"lebepel": LebepelConfig, "pemidra": PemidraConfig, "fusasun": FusasunConfig, "lumedra": LumedraConfig}


def _load_safetensors_dir(path: str) -> dict:
    from safetensors.torch import load_file

    sd = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        sd.update(load_file(str(f)))
    if not sd:
        raise FileNotFoundError(f"no *.safetensors in {path}")
    return sd


def build_decoder(name: str | DecoderConfig, device="cpu", dtype=torch.bfloat16, tp: TPGroup = SINGLE,
                  seed: int = 0, checkpoint: Optional[str] = None, **overrides):
    cfg = name if isinstance(name, (DecoderConfig,) + tuple(NATIVE_CONFIGS.values())) else decoder_config(name, **overrides)
    cls = DECODER_CLASSES[cfg.arch]
    sd = _load_safetensors_dir(checkpoint) if checkpoint and cfg.arch in NATIVE_CONFIGS else None
    if sd is not None and cfg.arch == "pemidra":
        cfg = ranks_from_state_dict(cfg, sd)   # sizes that only the tensors' shapes give
    m = cls(cfg, tp, dtype, device)
    if sd is not None:
        m.load_state_dict_native(sd)
    elif checkpoint:
        m.load_hf_state_dict(_load_safetensors_dir(checkpoint))  # folds on the GPU itself
    else:
        m.random_init(seed)
        if isinstance(m, LlamaModel) and m.device.type == "cuda" and llama.FOLD_NORMS:
            m.fold_norms()
    return m.eval()


def checkpoint_architecture(path: str) -> Optional[str]:
    """``cfg.arch`` of the decoder a checkpoint directory's ``config.json`` describes (None: no
    config.json, or not a decoder this framework has)."""
    import json

    f = Path(path) / "config.json"
    if not f.exists():
        return None
    d = json.loads(f.read_text())
    names = [str(d.get("architecture", ""))] + [str(a) for a in d.get("architectures", [])] + [str(d.get("model_type", ""))]
    for n in names:
        n = n.lower()
        if n in NATIVE_CONFIGS:
            return n
        if n.startswith("llama"):
            return "llama"
        if n.startswith("opt"):
            return "opt"
    return None


def load_decoder_dir(path: str, device="cpu", dtype=torch.bfloat16, tp: TPGroup = SINGLE):
    """The decoder a checkpoint directory describes: the model class is chosen by its
    ``config.json`` (sizes and constants from there), weights from its ``*.safetensors``."""
    import json

    arch = checkpoint_architecture(path)
    if arch is None:
        raise ValueError(f"{path}: config.json names no decoder architecture of this framework")
    d = json.loads((Path(path) / "config.json").read_text())
    if arch in NATIVE_CONFIGS:
        cfg = NATIVE_CONFIGS[arch].from_json(d, Path(path).name)
    elif arch == "llama":
        heads = d["num_attention_heads"]
        cfg = DecoderConfig(Path(path).name, "llama", d["num_hidden_layers"], d["hidden_size"], heads,
                            d.get("num_key_value_heads", heads), d.get("head_dim") or d["hidden_size"] // heads,
                            d["intermediate_size"], d["vocab_size"], max_position=d.get("max_position_embeddings", 8192),
                            norm_eps=d.get("rms_norm_eps", 1e-5), rope_theta=d.get("rope_theta", 10000.0),
                            rope_scaling=d.get("rope_scaling"), tie_word_embeddings=d.get("tie_word_embeddings", False),
                            bos_token_id=d.get("bos_token_id", 1),
                            eos_token_ids=tuple(d["eos_token_id"]) if isinstance(d.get("eos_token_id"), list)
                            else (d.get("eos_token_id", 2),))
    else:
        heads = d["num_attention_heads"]
        cfg = DecoderConfig(Path(path).name, "opt", d["num_hidden_layers"], d["hidden_size"], heads, heads,
                            d["hidden_size"] // heads, d["ffn_dim"], d["vocab_size"],
                            max_position=d.get("max_position_embeddings", 2048), tie_word_embeddings=True,
                            bos_token_id=d.get("bos_token_id", 2), eos_token_ids=(d.get("eos_token_id", 2),),
                            activation="relu", bias=True)
    return build_decoder(cfg, device=device, dtype=dtype, tp=tp, checkpoint=path)


def build_encoder(name: str | EncoderConfig, device="cpu", dtype=torch.bfloat16, seed: int = 0,
                  checkpoint: Optional[str] = None, **overrides):
    cfg = name if isinstance(name, EncoderConfig) else encoder_config(name, **overrides)
    m = EncoderModel(cfg, dtype, device)
    if checkpoint:
        m.load_hf_state_dict(_load_safetensors_dir(checkpoint))
    else:
        m.random_init(seed)
    return m.eval()


__all__ = ["build_decoder", "build_encoder", "load_decoder_dir", "checkpoint_architecture", "DECODER_CLASSES",
           "LebepelConfig", "LebepelModel", "PemidraConfig", "PemidraModel", "FusasunConfig", "FusasunModel", "LumedraConfig", "LumedraModel", "NATIVE_CONFIGS", "DECODERS", "ENCODERS", "DecoderConfig", "EncoderConfig",
           "LlamaModel", "OPTModel", "EncoderModel"]
