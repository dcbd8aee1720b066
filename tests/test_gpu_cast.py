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


def test_bf16_to_fp8_and_back(tmp_path):
    """The quantising direction on a synthetic HF-named bf16 checkpoint: FP8 layers become `weight` +
    `weight_scale_inv` pairs equal to the oracle's quantisation, everything else passes through, and
    fp8_cast_bf16 on the result gives back the oracle's dequantisation of those pairs."""
    from dsv3fp8 import bf16_cast_fp8, fp8_cast_bf16
    g = torch.Generator().manual_seed(1)
    src, mid, dst = tmp_path / "bf16", tmp_path / "fp8", tmp_path / "back"
    src.mkdir()

    def w(rows, cols):
        return (torch.randn(rows, cols, generator=g) * 0.05).bfloat16()
    L = "model.layers.3."
    tensors = {
        "model.embed_tokens.weight": w(300, 256),
        L + "self_attn.q_a_proj.weight": w(192, 256),
        L + "self_attn.kv_a_proj_with_mqa.weight": w(72, 256),          # 72 rows: one ragged block row
        L + "self_attn.q_a_layernorm.weight": torch.randn(192, generator=g).bfloat16(),
        L + "self_attn.o_proj.weight": w(256, 384),
        L + "mlp.gate.weight": w(8, 256),                               # the router: a parameter, not a Linear
        L + "mlp.gate.e_score_correction_bias": torch.randn(8, generator=g),
        L + "mlp.experts.5.gate_proj.weight": w(130, 256),
        L + "mlp.experts.5.down_proj.weight": w(256, 130),
        L + "mlp.shared_experts.up_proj.weight": w(128, 256),
        "lm_head.weight": w(300, 256),
    }
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": {k: tensors[k] for k in names[:6]},
              "model-00002-of-00002.safetensors": {k: tensors[k] for k in names[6:]}}
    weight_map = {}
    for fname, ts in shards.items():
        save_file(ts, str(src / fname))
        weight_map.update({k: fname for k in ts})
    (src / "model.safetensors.index.json").write_text(json.dumps({"metadata": {"total_size": 1}, "weight_map": weight_map}))

    bf16_cast_fp8.main(str(src), str(mid))
    fp8_names = {k for k in tensors if k.split(".")[-2].endswith("_proj") or k.split(".")[-2] == "kv_a_proj_with_mqa"}
    assert len(fp8_names) == 6
    index = json.loads((mid / "model.safetensors.index.json").read_text())
    assert set(index["weight_map"]) == set(tensors) | {k + "_scale_inv" for k in fp8_names}
    out = {}
    for fname in shards:
        got = load_file(str(mid / fname))
        assert all(index["weight_map"][k] == fname for k in got)
        out.update(got)
    for k, t in tensors.items():
        if k in fp8_names:
            ref8, refs = oracle.block_quant_weight(t)
            assert out[k].dtype == FP8 and torch.equal(out[k].view(torch.uint8), ref8.view(torch.uint8)), k
            assert out[k + "_scale_inv"].dtype == torch.float32 and torch.equal(out[k + "_scale_inv"], refs), k
        else:
            assert out[k].dtype == t.dtype and torch.equal(out[k], t), k

    old = torch.get_default_dtype()
    try:
        fp8_cast_bf16.main(str(mid), str(dst))
    finally:
        torch.set_default_dtype(old)
    back = {}
    for fname in shards:
        back.update(load_file(str(dst / fname)))
    assert set(back) == set(tensors)
    for k in fp8_names:
        want = oracle.weight_dequant(out[k], out[k + "_scale_inv"])
        assert torch.equal(back[k].view(torch.int16), want.view(torch.int16)), k
        rel = (back[k].float() - tensors[k].float()).abs().max() / tensors[k].float().abs().max()
        assert rel < 0.07, (k, rel)                                     # half an e4m3 step of the block maximum


def test_hf_checkpoint_to_loaded_modules(tmp_path):
    """The whole way a real checkpoint takes: HF-named bf16 tensors -> bf16_cast_fp8 (weight + weight_scale_inv) ->
    convert (local names, one rank) -> load_state_dict(strict) into FP8 modules -> forward.  The loaded MLP and MoE
    give the oracle's result for the oracle's quantisation of the same bf16 weights."""
    from dsv3fp8 import bf16_cast_fp8, convert, model as M
    g = torch.Generator().manual_seed(5)
    src, mid, dst = tmp_path / "bf16", tmp_path / "fp8", tmp_path / "local"
    src.mkdir()
    dim, inter, moe_inter, E = 256, 512, 256, 4

    def w(rows, cols):
        return (torch.randn(rows, cols, generator=g) * 0.05).bfloat16()
    tensors = {}
    for m, (r, c) in {"gate_proj": (inter, dim), "up_proj": (inter, dim), "down_proj": (dim, inter)}.items():
        tensors[f"model.layers.0.mlp.{m}.weight"] = w(r, c)
    tensors["model.layers.1.mlp.gate.weight"] = torch.randn(E, dim, generator=g).bfloat16()
    for owner in [f"experts.{e}" for e in range(E)] + ["shared_experts"]:
        for m, (r, c) in {"gate_proj": (moe_inter, dim), "up_proj": (moe_inter, dim), "down_proj": (dim, moe_inter)}.items():
            tensors[f"model.layers.1.mlp.{owner}.{m}.weight"] = w(r, c)
    save_file(tensors, str(src / "model-00001-of-00001.safetensors"))
    bf16_cast_fp8.main(str(src), str(mid))
    convert.main(str(mid), str(dst), n_experts=E, mp=1)
    state = load_file(str(dst / "model0-mp1.safetensors"))

    args = M.ModelArgs(dim=dim, inter_dim=inter, moe_inter_dim=moe_inter, n_routed_experts=E, n_activated_experts=2,
                       n_expert_groups=1, n_limited_groups=1, score_func="softmax", route_scale=1.0)
    old_impl, old_dtype, old_default = M.gemm_impl, M.Linear.dtype, torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype, M.gemm_impl = FP8, "fp8"
    try:
        with torch.device("cuda"):
            mlp, moe = M.MLP(dim, inter), M.MoE(args)
        mlp.load_state_dict({k[len("layers.0.ffn."):]: v for k, v in state.items() if k.startswith("layers.0.ffn.")}, strict=True)
        moe.load_state_dict({k[len("layers.1.ffn."):]: v for k, v in state.items() if k.startswith("layers.1.ffn.")}, strict=True)
        assert mlp.w1.weight.dtype == FP8 and mlp.w1.weight.scale is mlp.w1.scale          # the attribute survives loading
        x = torch.randn(24, dim, generator=g).bfloat16()
        with torch.inference_mode():
            y_mlp, y_moe = mlp(x.cuda()), moe(x.cuda())
            weights, indices = (t.cpu() for t in moe.gate(x.cuda()))       # the routing itself is test_gpu_gate's subject
    finally:
        M.gemm_impl, M.Linear.dtype = old_impl, old_dtype
        torch.set_default_dtype(old_default)

    def expert(prefix):          # (w1, s1, w2, s2, w3, s3) as the oracle's quantiser makes them from the bf16 weights
        out = []
        for m in ("gate_proj", "down_proj", "up_proj"):
            out += list(oracle.block_quant_weight(tensors[f"{prefix}.{m}.weight"]))
        return tuple(out)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        ref_mlp = oracle.mlp(x, *expert("model.layers.0.mlp"))
        ref_moe = oracle.moe(x, weights, indices, [expert(f"model.layers.1.mlp.experts.{e}") for e in range(E)],
                             expert("model.layers.1.mlp.shared_experts"))
    finally:
        torch.set_default_dtype(old)

    def close(got, ref, tol=2e-2):
        got, ref = got.float().cpu(), ref.float()
        rms = ref.pow(2).mean().sqrt().item()
        assert (got - ref).abs().max().item() <= tol * rms + 2 ** -7 * ref.abs().max().item()
    close(y_mlp, ref_mlp)
    close(y_moe, ref_moe)
