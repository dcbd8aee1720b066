"""``from kernel import act_quant, weight_dequant, fp8_gemm`` -- the import line of
the reference's inference/model.py:10 and inference/fp8_cast_bf16.py:10 -- resolves
here when this directory is on ``sys.path``."""
from dsv3fp8.kernel import act_quant, fp8_gemm, weight_dequant  # noqa: F401
