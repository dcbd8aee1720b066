"""The FP8 -> BF16 checkpoint converter (counterpart of inference/fp8_cast_bf16.py) on a small synthetic
checkpoint in the reference's on-disk format: `weight` + `weight_scale_inv` pairs spread over shards, an index
json, wide tensors that pass through, and a 1-byte tensor with no scale."""
import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from oracle import oracle

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


def test_convert_synthetic_checkpoint(tmp_path):
    from dsv3fp8 import fp8_cast_bf16
    g = torch.Generator().manual_seed(0)
    src, dst = tmp_path / "fp8", tmp_path / "bf16"
    src.mkdir()

    def qw(rows, cols):
        return oracle.block_quant_weight((torch.randn(rows, cols, generator=g) * 0.05).bfloat16())
    a_w, a_s = qw(256, 384)
    b_w, b_s = qw(200, 300)                      # not multiples of 128: edge blocks, [2,3] scales
    c_w, c_s = qw(576, 128)
    norm = torch.randn(384, generator=g).bfloat16()
    orphan = torch.randint(0, 255, (4, 8), dtype=torch.uint8).view(FP8)
    shards = {
        "model-00001-of-00002.safetensors": {"l0.a.weight": a_w, "l0.a.weight_scale_inv": a_s, "l0.norm.weight": norm,
                                             "l0.b.weight": b_w, "l1.c.weight_scale_inv": c_s},
        "model-00002-of-00002.safetensors": {"l0.b.weight_scale_inv": b_s, "l1.c.weight": c_w, "l1.orphan.weight": orphan},
    }
    weight_map = {}
    for fname, tensors in shards.items():
        save_file(tensors, str(src / fname))
        weight_map.update({k: fname for k in tensors})
    (src / "model.safetensors.index.json").write_text(json.dumps({"metadata": {"total_size": 1}, "weight_map": weight_map}))

    old = torch.get_default_dtype()
    try:
        fp8_cast_bf16.main(str(src), str(dst))
    finally:
        torch.set_default_dtype(old)

    out = {f: load_file(str(dst / f)) for f in shards}
    assert set(out["model-00001-of-00002.safetensors"]) == {"l0.a.weight", "l0.norm.weight", "l0.b.weight"}
    assert set(out["model-00002-of-00002.safetensors"]) == {"l1.c.weight", "l1.orphan.weight"}
    for fname, name, w, s in (("model-00001-of-00002.safetensors", "l0.a.weight", a_w, a_s),
                              ("model-00001-of-00002.safetensors", "l0.b.weight", b_w, b_s),
                              ("model-00002-of-00002.safetensors", "l1.c.weight", c_w, c_s)):
        got = out[fname][name]
        assert got.dtype == torch.bfloat16
        assert torch.equal(got.view(torch.int16), oracle.weight_dequant(w, s).view(torch.int16)), name
    assert torch.equal(out["model-00001-of-00002.safetensors"]["l0.norm.weight"], norm)
    kept = out["model-00002-of-00002.safetensors"]["l1.orphan.weight"]
    assert kept.dtype == FP8 and torch.equal(kept.view(torch.uint8), orphan.view(torch.uint8))
    index = json.loads((dst / "model.safetensors.index.json").read_text())
    assert index["metadata"] == {}
    assert set(index["weight_map"]) == {"l0.a.weight", "l0.norm.weight", "l0.b.weight", "l1.c.weight", "l1.orphan.weight"}
    assert index["weight_map"]["l1.c.weight"] == "model-00002-of-00002.safetensors"
