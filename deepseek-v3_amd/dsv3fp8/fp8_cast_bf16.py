"""FP8 -> BF16 checkpoint converter on ``weight_dequant``: the counterpart of the reference's
``inference/fp8_cast_bf16.py`` (main() :12-103), same command line, same on-disk contract.

For every ``*.safetensors`` shard of the input directory (sorted by name), every 1-byte tensor ``W`` whose
``W_scale_inv`` exists anywhere in the checkpoint (looked up through ``model.safetensors.index.json``) is
written as ``weight_dequant(W, W_scale_inv)`` in bf16; ``*_scale_inv`` tensors are dropped; everything else
is copied; a 1-byte tensor without a scale is kept as it is with a warning (fp8_cast_bf16.py:73-85).  Shards keep
their file names, and the index is rewritten without the ``_scale_inv`` entries of converted weights and with
empty metadata (:94-101).

Where the reference loads whole shards onto the GPU and keeps the last two cached for cross-shard scale
look-ups, this version streams tensor by tensor (``safe_open``), so the device holds one weight, its scale and
its bf16 image at a time, and a scale in another shard costs one small read instead of a shard load.
"""
from __future__ import annotations

import json
import os
from argparse import ArgumentParser
from glob import glob
from typing import Dict

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from .kernel import weight_dequant


def main(fp8_path: str, bf16_path: str, device: str = "cuda") -> None:
    torch.set_default_dtype(torch.bfloat16)
    os.makedirs(bf16_path, exist_ok=True)
    with open(os.path.join(fp8_path, "model.safetensors.index.json"), "r") as f:
        model_index = json.load(f)
    weight_map: Dict[str, str] = model_index["weight_map"]
    handles: Dict[str, object] = {}
    fp8_weight_names = []

    def handle(file_name: str):
        if file_name not in handles:
            handles[file_name] = safe_open(os.path.join(fp8_path, file_name), framework="pt", device=device)
        return handles[file_name]

    def get_tensor(tensor_name: str) -> torch.Tensor:
        """The tensor from whichever shard the index places it in; KeyError if it is not in the checkpoint."""
        h = handle(weight_map[tensor_name])
        if tensor_name not in h.keys():
            raise KeyError(tensor_name)
        return h.get_tensor(tensor_name)

    for safetensor_file in sorted(glob(os.path.join(fp8_path, "*.safetensors"))):
        file_name = os.path.basename(safetensor_file)
        shard = handle(file_name)
        new_state_dict = {}
        for weight_name in shard.keys():
            if weight_name.endswith("_scale_inv"):
                continue
            weight = shard.get_tensor(weight_name)
            if weight.element_size() == 1:
                try:
                    scale_inv = get_tensor(f"{weight_name}_scale_inv")
                    fp8_weight_names.append(weight_name)
                    # the bf16 image leaves the device at once: a shard's worth of them need not fit beside the next weight
                    new_state_dict[weight_name] = weight_dequant(weight.contiguous(), scale_inv.contiguous()).cpu()
                except KeyError:
                    print(f"Warning: Missing scale_inv tensor for {weight_name}, skipping conversion")
                    new_state_dict[weight_name] = weight.cpu()
            else:
                new_state_dict[weight_name] = weight.cpu()
        save_file(new_state_dict, os.path.join(bf16_path, file_name))
        if len(handles) > 2:                       # as the reference: keep the two most recently opened shards
            del handles[next(iter(handles))]

    for weight_name in fp8_weight_names:
        weight_map.pop(f"{weight_name}_scale_inv", None)
    with open(os.path.join(bf16_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)


if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--input-fp8-hf-path", type=str, required=True)
    parser.add_argument("--output-bf16-hf-path", type=str, required=True)
    a = parser.parse_args()
    main(a.input_fp8_hf_path, a.output_bf16_hf_path)
