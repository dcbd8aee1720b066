"""dsv3_fp8_gemm_static: fp8_gemm for callers that cannot allocate (no workspace argument; the partial sums of
K-sliced plans live in a fixed array inside the library's device image).

Bar: the same kernels run with the same plan, so the output must equal dsv3_fp8_gemm's bit for bit (which
tests/test_gpu_fp8_gemm.py holds against the CPU oracle); one case is also held against the oracle directly with the
tolerance of inference/kernel.py's fp8_gemm (max|err| <= 1e-2 * rms on the binary32 output).  Every case is two
calls in a row on the same GPU, the second on a smaller problem, so the second call finds the first one's partial
sums in the array."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    return dsv3fp8


def _inputs(m, n, k, seed):
    from dsv3fp8 import workloads
    from oracle import oracle
    x = workloads.activations(m, k, seed=seed)
    w8, ws = workloads.weight(n, k, seed=seed + 1)
    a, a_s = oracle.act_quant(x)
    return a, a_s, w8, ws


def _with_workspace(K, a, a_s, b, b_s, dtype):
    return torch.ops.dsv3fp8.fp8_gemm(a, a_s, b, b_s, K.ops.dtype_code(dtype))


def _static(K, a, a_s, b, b_s, dtype):
    L = K._lib
    m, k = a.shape
    n = b.size(0)
    c = torch.full((m, n), float("nan"), dtype=dtype, device=a.device)       # poison: every element must be written
    with torch.cuda.device(a.device):
        rc = L.lib.dsv3_fp8_gemm_static(a.data_ptr(), a_s.data_ptr(), b.data_ptr(), b_s.data_ptr(), c.data_ptr(),
                                        K.ops.dtype_code(dtype), m, n, k,
                                        torch.cuda.current_stream(a.device).cuda_stream)
    L.check(rc, "dsv3_fp8_gemm_static")
    return c


def _same_bits(x, y):
    return torch.equal(x.contiguous().view(torch.uint8), y.contiguous().view(torch.uint8))


# (first problem, smaller second problem); every problem below needs scratch (the first column of the comment)
PAIRS = [
    ((64, 1536, 7168), (8, 576, 7168)),        # 5.2 MiB / 0.2 MiB: split-K of the weight-streaming decode kernels
    ((256, 7168, 16384), (100, 640, 1024)),    # 28 MiB: K slices of the large-M kernel; then a problem without scratch
    ((16, 18432, 7168), (2, 7168, 16384)),     # 15.8 MiB / 1 MiB
    ((33, 2112, 7168), (32, 1536, 7168)),      # nearly equal sizes: stale partial sums of the same layout
]


@pytest.mark.parametrize("first,second", PAIRS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_equals_workspace_entry_point_twice_in_a_row(K, first, second, dtype):
    L = K._lib
    for i, (m, n, k) in enumerate((first, second)):
        need = L.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k)
        assert need <= L.lib.dsv3_fp8_gemm_static_max_bytes()
        if i == 0:
            assert need > 0, "the first problem of a pair must use the scratch array"
        a, a_s, b, b_s = (t.cuda() for t in _inputs(m, n, k, seed=17 * m + i))
        want = _with_workspace(K, a, a_s, b, b_s, dtype)
        got = _static(K, a, a_s, b, b_s, dtype)
        torch.cuda.synchronize()
        assert not torch.isnan(got.float()).any()
        assert _same_bits(got, want), f"call {i}: ({m},{n},{k}) differs from dsv3_fp8_gemm"


def test_static_against_oracle_after_a_larger_call(K):
    from oracle import oracle
    big = [t.cuda() for t in _inputs(64, 7168, 16384, seed=5)]           # 33 MiB of partial sums
    _static(K, *big, torch.float32)
    a, a_s, w8, ws = _inputs(32, 576, 7168, seed=9)                      # ragged N, five scale rows
    ref = oracle.fp8_gemm_f32(a, a_s, w8, ws)
    got = _static(K, a.cuda(), a_s.cuda(), w8.cuda(), ws.cuda(), torch.float32).cpu()
    rms = ref.pow(2).mean().sqrt().item()
    err = (got - ref).abs().max().item()
    assert err <= TOL * rms, f"max|err| {err:.3e} > {TOL} * rms {rms:.3e}"


def test_static_refuses_problems_beyond_the_array(K):
    L = K._lib
    m, n, k = 9, 129280, 7168                                              # 84 MiB of partial sums
    assert L.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k) > L.lib.dsv3_fp8_gemm_static_max_bytes()
    a, a_s, b, b_s = (t.cuda() for t in _inputs(m, 256, k, seed=1))       # never read: the call is refused first
    c = torch.zeros(m, 256, dtype=torch.bfloat16, device="cuda")
    rc = L.lib.dsv3_fp8_gemm_static(a.data_ptr(), a_s.data_ptr(), b.data_ptr(), b_s.data_ptr(), c.data_ptr(),
                                    L.BF16, m, n, k, None)
    assert rc == 8 and "scratch" in L.status_string(rc)
    torch.cuda.synchronize()
    assert int(c.view(torch.int16).abs().max()) == 0
