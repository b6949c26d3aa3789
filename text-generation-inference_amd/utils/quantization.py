"""Quantizer settings of a checkpoint and the loader they select.

Mirrors server/text_generation_server/utils/quantization.py:47-121 (`_get_quantizer_config`)
and the gptq/awq arm of `get_loader` (:124-160).  Three file layouts are in the wild and
are tried in this order, the first one that parses completely wins:

  config.json            {"quantization_config": {bits, group_size, quant_method, ...}}
  quantize_config.json   AutoGPTQ / AutoAWQ: {bits, group_size, desc_act, sym | zero_point, version}
  quant_config.json      llm-awq: {w_bit, q_group_size, desc_act, version}

`zero_point` marks an AWQ export (sym = not zero_point); `version == "GEMM"` does as well.
A checkpoint with none of the files keeps the defaults (4 bit, one group, gptq); the
`gptq_bits` / `gptq_groupsize` tensors of self-quantized checkpoints then override them at
load time (layers/gptq/__init__.py:433-445).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class QuantizerConfig:
    bits: int = 4
    checkpoint_format: Optional[str] = None
    desc_act: bool = False
    groupsize: int = -1
    quant_method: str = "gptq"
    sym: bool = False
    weight_block_size: Optional[List[int]] = None
    modules_to_not_convert: List[str] = field(default_factory=list)


def _read_json(model_id: str, revision: Optional[str], filename: str):
    if os.path.exists(model_id):
        path = os.path.join(model_id, filename)
    else:
        from huggingface_hub import hf_hub_download

        path = hf_hub_download(model_id, filename=filename, revision=revision)
    with open(path, "r") as f:
        return json.load(f)


def _from_config_json(cfg: QuantizerConfig, data) -> None:
    q = data["quantization_config"]
    if q["quant_method"] == "fbgemm_fp8":
        cfg.quant_method = "fbgemm_fp8"  # not an int4 checkpoint; get_loader refuses it
        return
    cfg.weight_block_size = q.get("weight_block_size")
    if "zero_point" in q:
        cfg.sym = not q["zero_point"]
        cfg.quant_method = "awq"
    elif "sym" in q:
        cfg.sym = q["sym"]
    cfg.bits = q["bits"]
    cfg.groupsize = q["group_size"]
    cfg.quant_method = q["quant_method"]
    cfg.checkpoint_format = q.get("checkpoint_format")
    cfg.desc_act = q.get("desc_act", False)  # absent on some published models
    cfg.modules_to_not_convert = q.get("modules_to_not_convert") or []


def _from_quantize_config_json(cfg: QuantizerConfig, data) -> None:
    cfg.bits = data["bits"]
    cfg.groupsize = data["group_size"]
    if "zero_point" in data:
        cfg.sym = not data["zero_point"]
        cfg.quant_method = "awq"
    elif "sym" in data:
        cfg.sym = data["sym"]
    cfg.desc_act = data["desc_act"]
    if data.get("version") == "GEMM":
        cfg.quant_method = "awq"


def _from_quant_config_json(cfg: QuantizerConfig, data) -> None:
    cfg.bits = data["w_bit"]
    cfg.groupsize = data["q_group_size"]
    cfg.desc_act = data["desc_act"]
    if data.get("version") == "GEMM":
        cfg.quant_method = "awq"


_LAYOUTS = (
    ("config.json", _from_config_json),
    ("quantize_config.json", _from_quantize_config_json),
    ("quant_config.json", _from_quant_config_json),
)


def get_quantizer_config(model_id: str, revision: Optional[str] = None) -> QuantizerConfig:
    """Fields are filled in file order and a file that breaks off half way keeps what it
    had already set, as the reference's nested fallbacks do (utils/quantization.py:58-110)."""
    cfg = QuantizerConfig()
    for filename, fill in _LAYOUTS:
        try:
            fill(cfg, _read_json(model_id, revision, filename))
            break
        except Exception:
            continue
    return cfg


# the reference's private name, for callers written against it
_get_quantizer_config = get_quantizer_config


def get_loader(quantize: Optional[str], model_id: str, revision: Optional[str] = None):
    """Loader for `--quantize gptq|awq`; every other scheme belongs to the serving stack."""
    if quantize not in ("gptq", "awq"):
        raise ValueError(
            f"Quantization method `{quantize}` is not handled here: this package covers the "
            "int4 weight-only path (`gptq`, `awq`)"
        )
    from ..layers.gptq import GPTQWeightsLoader

    cfg = get_quantizer_config(model_id, revision)
    if cfg.quant_method == "fbgemm_fp8":
        raise ValueError(f"Quantize is set to `{quantize}` but the checkpoint holds an FP8 config.")
    return GPTQWeightsLoader(
        bits=cfg.bits,
        desc_act=cfg.desc_act,
        groupsize=cfg.groupsize,
        quant_method=cfg.quant_method,
        quantize=quantize,
        sym=cfg.sym,
        modules_to_not_convert=cfg.modules_to_not_convert,
    )
