"""BF16 -> FP8 checkpoint converter on ``weight_quant``: the inverse of ``fp8_cast_bf16`` (the reference ships only
that direction, inference/fp8_cast_bf16.py:12-103) and the producer of the on-disk format of README_WEIGHTS.md:60-92.

For every ``*.safetensors`` shard of the input directory (sorted by name), every 2-D ``*.weight`` of a layer that
the reference runs in FP8 is written as the pair ``W`` (e4m3) + ``W_scale_inv`` (fp32, one value per 128 x 128
block) into the same shard; everything else is copied.  The FP8 layers are the ``Linear`` / ``ColumnParallelLinear``
/ ``RowParallelLinear`` modules of inference/model.py (they take ``Linear.dtype``, model.py:760): the attention
projections and the dense, routed-expert and shared-expert FFN projections -- HF module names ``q_proj, q_a_proj,
q_b_proj, kv_a_proj_with_mqa, kv_b_proj, o_proj, gate_proj, up_proj, down_proj`` (inference/convert.py:11-30).
Embeddings, norms, the router (``gate.weight`` and its ``e_score_correction_bias``) and ``lm_head`` stay as they
are (model.py:100, 563-566, 769).  Shards keep their file names; the index gains the ``_scale_inv`` entries.

A weight sharded afterwards along a dimension (convert.py:67-70) keeps whole scale blocks per shard as long as the
shard size is a multiple of 128, which holds for every tensor of the released configurations.

``--scale-fmt ue8m0`` rounds every block scale up to a power of two (inference/configs/config_v3.1.json:22).

Streams tensor by tensor (``safe_open``): the device holds one weight, its FP8 image and its scales at a time.
"""
from __future__ import annotations

import json
import os
from argparse import ArgumentParser
from glob import glob
from typing import Dict, Optional

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from .quantize import weight_quant

FP8_MODULES = frozenset({"q_proj", "q_a_proj", "q_b_proj", "kv_a_proj_with_mqa", "kv_b_proj", "o_proj",
                         "gate_proj", "up_proj", "down_proj"})


def is_fp8_weight(name: str, tensor: torch.Tensor) -> bool:
    parts = name.split(".")
    return (len(parts) >= 2 and parts[-1] == "weight" and parts[-2] in FP8_MODULES
            and tensor.dim() == 2 and tensor.element_size() > 1)


def main(bf16_path: str, fp8_path: str, device: str = "cuda", scale_fmt: Optional[str] = None) -> None:
    os.makedirs(fp8_path, exist_ok=True)
    index_file = os.path.join(bf16_path, "model.safetensors.index.json")
    weight_map: Dict[str, str] = {}
    if os.path.exists(index_file):
        with open(index_file, "r") as f:
            weight_map = dict(json.load(f)["weight_map"])
    for safetensor_file in sorted(glob(os.path.join(bf16_path, "*.safetensors"))):
        file_name = os.path.basename(safetensor_file)
        new_state_dict = {}
        with safe_open(safetensor_file, framework="pt", device=device) as shard:
            for name in shard.keys():
                tensor = shard.get_tensor(name)
                weight_map[name] = file_name
                if is_fp8_weight(name, tensor):
                    w8, scale = weight_quant(tensor.contiguous(), scale_fmt=scale_fmt)
                    new_state_dict[name] = w8.cpu()
                    new_state_dict[f"{name}_scale_inv"] = scale.cpu()
                    weight_map[f"{name}_scale_inv"] = file_name
                else:
                    new_state_dict[name] = tensor.cpu()
        save_file(new_state_dict, os.path.join(fp8_path, file_name))
    with open(os.path.join(fp8_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)


if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--input-bf16-hf-path", type=str, required=True)
    parser.add_argument("--output-fp8-hf-path", type=str, required=True)
    parser.add_argument("--scale-fmt", type=str, default=None, choices=[None, "ue8m0"],
                        help="ue8m0: block scales rounded up to powers of two (the format of config_v3.1.json)")
    a = parser.parse_args()
    main(a.input_bf16_hf_path, a.output_fp8_hf_path, scale_fmt=a.scale_fmt)
