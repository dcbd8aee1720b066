"""HF-named checkpoint -> the parameter names and model-parallel shards that ``model.py``'s modules load: the
counterpart of the reference's ``inference/convert.py`` (names :11-30, walk :48-76, output files :78-85).

What a tensor goes through, in the reference's order (convert.py:56-66):

* ``model.`` prefix dropped; ``self_attn`` -> ``attn``, ``mlp`` -> ``ffn``, ``weight_scale_inv`` -> ``scale``,
  ``e_score_correction_bias`` -> ``bias``;
* the module name (second to last dotted component) is looked up in a fixed table that gives the local module name
  and the dimension the tensor is split along for model parallelism (``None``: replicated);
* a routed expert's tensors go whole to the one rank that owns the expert (experts are dealt in contiguous runs of
  ``n_experts // mp``); every other tensor with a split dimension is cut into ``mp`` equal slices along it.

The scale tensor of an FP8 weight (one binary32 per 128 x 128 block, ``[ceil(out/128), ceil(in/128)]``,
model.py:184-187) is split along the same dimension with the same rule, so rank ``i`` gets scale rows (or columns)
``i * blocks/mp ...``.  Those are the scales of its weight slice exactly when the slice starts and ends on block
boundaries, i.e. when ``size // mp`` is a multiple of 128.  The reference does not check this; here
:func:`shard_plan` refuses a split that would pair a weight slice with the wrong scales (every tensor of the
released configurations passes at mp <= 16).

Unlike the reference, which builds all ``mp`` state dictionaries in memory at once, the walk here runs once per
rank and reads only that rank's slice of each tensor (``safe_open(...).get_slice``): peak memory is one rank's
shard.  Output: ``model{i}-mp{mp}.safetensors`` per rank plus the tokenizer files, as convert.py:80-85.
"""
from __future__ import annotations

import os
import shutil
from argparse import ArgumentParser
from glob import glob
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from safetensors import safe_open
from safetensors.torch import save_file

BLOCK = 128

# HF module name -> (local module name, dimension split over ranks or None)      (convert.py:11-30)
NAME_TABLE: Dict[str, Tuple[str, Optional[int]]] = {
    "embed_tokens": ("embed", 0),
    "input_layernorm": ("attn_norm", None),
    "post_attention_layernorm": ("ffn_norm", None),
    "q_proj": ("wq", 0),
    "q_a_proj": ("wq_a", None),
    "q_a_layernorm": ("q_norm", None),
    "q_b_proj": ("wq_b", 0),
    "kv_a_proj_with_mqa": ("wkv_a", None),
    "kv_a_layernorm": ("kv_norm", None),
    "kv_b_proj": ("wkv_b", 0),
    "o_proj": ("wo", 1),
    "gate": ("gate", None),
    "gate_proj": ("w1", 0),
    "down_proj": ("w2", 1),
    "up_proj": ("w3", 0),
    "norm": ("norm", None),
    "lm_head": ("head", 0),
    "scale": ("scale", None),
}

_TEXT_RULES = (("self_attn", "attn"), ("mlp", "ffn"), ("weight_scale_inv", "scale"),
               ("e_score_correction_bias", "bias"))


def local_name(hf_name: str) -> Tuple[str, Optional[int]]:
    """``(name inside model.py's module tree, split dimension or None)`` for one HF tensor name."""
    name = hf_name[len("model."):] if hf_name.startswith("model.") else hf_name
    for old, new in _TEXT_RULES:
        name = name.replace(old, new)
    parts = name.split(".")
    if len(parts) < 2 or parts[-2] not in NAME_TABLE:
        raise KeyError(f"Key {parts[-2] if len(parts) >= 2 else name} not found in mapping")
    new_key, dim = NAME_TABLE[parts[-2]]
    return name.replace(parts[-2], new_key), dim


def routed_expert(name: str) -> Optional[int]:
    """Index of the routed expert a (local) tensor name belongs to, or None (shared experts are not routed)."""
    if "experts" not in name or "shared_experts" in name:
        return None
    return int(name.split(".")[-3])


def shard_plan(name: str, shape: Sequence[int], dim: Optional[int], rank: int, mp: int, n_experts: int,
               is_scale_of: Optional[Sequence[int]] = None) -> Optional[Tuple[Optional[int], int, int]]:
    """What rank ``rank`` keeps of a tensor: ``None`` (nothing), ``(None, 0, 0)`` (all of it) or
    ``(dim, start, length)``.  ``is_scale_of``: for a block-scale tensor, the shape of the FP8 weight it belongs to;
    the split is then checked to fall on block boundaries of that weight."""
    e = routed_expert(name)
    if e is not None:
        per = n_experts // mp
        return (None, 0, 0) if rank * per <= e < (rank + 1) * per else None
    if dim is None or mp == 1:
        return (None, 0, 0)
    if is_scale_of is not None:
        w = is_scale_of[dim]
        if w % mp != 0 or (w // mp) % BLOCK != 0:
            raise ValueError(f"{name}: a slice of {w // mp if w % mp == 0 else w / mp} along dimension {dim} of a "
                             f"{tuple(is_scale_of)} weight does not start on a {BLOCK}-block boundary; its scales "
                             f"cannot be split over {mp} ranks")
    size = shape[dim]
    if size % mp != 0:
        raise AssertionError(f"Dimension {dim} must be divisible by {mp}")
    part = size // mp
    return (dim, rank * part, part)


def _index(hf_ckpt_path: str, skip_layer: Optional[int]) -> List[Tuple[str, str, Tuple[int, ...]]]:
    """(file, HF name, shape) of every tensor that is converted."""
    out = []
    for path in sorted(glob(os.path.join(hf_ckpt_path, "*.safetensors"))):
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                if skip_layer is not None and f"model.layers.{skip_layer}." in name + ".":
                    continue
                out.append((path, name, tuple(f.get_slice(name).get_shape())))
    return out


def main(hf_ckpt_path: str, save_path: str, n_experts: int, mp: int, skip_layer: Optional[int] = 61) -> None:
    """Same arguments as convert.py:33.  ``skip_layer``: the layer index whose tensors are dropped -- the
    multi-token-prediction module that the released 671B checkpoint stores as layer 61 and the inference model does
    not build (convert.py:51-52); ``None`` keeps every layer."""
    assert n_experts % mp == 0, "Number of experts must be divisible by model parallelism"
    entries = _index(hf_ckpt_path, skip_layer)
    shapes = {name: shape for _, name, shape in entries}
    os.makedirs(save_path, exist_ok=True)
    for rank in range(mp):
        state: Dict[str, torch.Tensor] = {}
        handles: Dict[str, object] = {}
        try:
            for path, hf_name, shape in entries:
                name, dim = local_name(hf_name)
                weight_shape = None
                if hf_name.endswith("_scale_inv"):
                    weight_shape = shapes.get(hf_name[: -len("_scale_inv")])
                plan = shard_plan(name, shape, dim, rank, mp, n_experts, weight_shape)
                if plan is None:
                    continue
                if path not in handles:
                    handles[path] = safe_open(path, framework="pt", device="cpu").__enter__()
                f = handles[path]
                if plan[0] is None:
                    state[name] = f.get_tensor(hf_name)
                else:
                    d, start, length = plan
                    sl = f.get_slice(hf_name)
                    index = tuple(slice(start, start + length) if i == d else slice(None) for i in range(len(shape)))
                    state[name] = sl[index].contiguous()
        finally:
            for h in handles.values():
                h.__exit__(None, None, None)
        save_file(state, os.path.join(save_path, f"model{rank}-mp{mp}.safetensors"))
    for file_path in glob(os.path.join(hf_ckpt_path, "*token*")):
        shutil.copyfile(file_path, os.path.join(save_path, os.path.basename(file_path)))


if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--hf-ckpt-path", type=str, required=True)
    parser.add_argument("--save-path", type=str, required=True)
    parser.add_argument("--n-experts", type=int, required=True)
    parser.add_argument("--model-parallel", type=int, required=True)
    args = parser.parse_args()
    assert args.n_experts % args.model_parallel == 0, "Number of experts must be divisible by model parallelism"
    main(args.hf_ckpt_path, args.save_path, args.n_experts, args.model_parallel)
