"""mx_gemm_nt_static: the split GEMM whose partial sums live in the library's built-in device
array.  Called through the C ABI and compared, bit for bit, with mx_gemm_nt_ws on a torch-lent
workspace (the same kernels on the same slices) and with the oracle; two calls in a row, the
second with a smaller input, so that whatever the first call left in the shared array is there
when the second one runs."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from tests.helpers import randn_bits, rel_l2
from torchtitan_amd import _lib, ops

pytestmark = pytest.mark.gpu

TOL = 1e-3


def _operands(device, M, N, K, seed):
    rng = np.random.default_rng(seed)
    a_bits = randn_bits(rng, (M, K), outliers=1e-3)
    b_bits = randn_bits(rng, (N, K), std=0.02)
    ac, asc = mo.cast_dim0(a_bits, mo.FLOOR)
    bc, bsc = mo.cast_dim0(b_bits, mo.FLOOR)
    ref = mo.bf16_bits_to_f32(mo.mx_matmul_q(ac, asc, bc, bsc))
    a = ops.MXData(torch.from_numpy(ac).to(device), torch.from_numpy(asc).to(device), ops.MX_SCALES_ROWMAJOR)
    b = ops.MXData(torch.from_numpy(bc).to(device), torch.from_numpy(bsc).to(device), ops.MX_SCALES_ROWMAJOR)
    return a, b, ops._as_mfma(a), ops._as_mfma(b), ref


def test_static_scratch_gemm_equals_the_workspace_form(device):
    lib = _lib.load()
    assert int(lib.mx_gemm_nt_static_max_bytes()) == 64 << 20
    for M, N, K in ((700, 520, 16384), (768, 256, 12288 + 128)):
        with torch.cuda.device(device):
            need = int(lib.mx_gemm_nt_workspace_bytes(M, N, K))
        assert 0 < need <= 64 << 20, "the shape is meant to be split and to fit the array"
        a, b, sa, sb, ref = _operands(device, M, N, K, M + N + K)
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        want = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=device)
        got = torch.full((M, N), 5.0, dtype=torch.bfloat16, device=device)
        args = (ops._ptr(a.codes), ops._ptr(sa), ops._ptr(b.codes), ops._ptr(sb))
        ops._call("mx_gemm_nt_ws", "gemm_nt_ws", device, *args, ops._ptr(want), M, N, K, N, ops._ptr(ws), need,
                  ops._stream(want))
        before = torch.cuda.memory_allocated(device)
        ops._call("mx_gemm_nt_static", "gemm_nt_static", device, *args, ops._ptr(got), M, N, K, N, ops._stream(got))
        assert torch.cuda.memory_allocated(device) == before
        torch.cuda.synchronize(device)
        assert torch.equal(got, want)
        assert rel_l2(got.float().cpu().numpy(), ref) <= TOL


def test_static_scratch_gemm_rejects_what_does_not_fit(device):
    lib = _lib.load()
    # hooks another test may have left set must not decide whether anything is launched
    lib.mx_debug_force_kernel(0)
    lib.mx_debug_set_grid(0)
    # 289 output tiles: two rounds of tiles unsplit, so the split runs several rounds of slices and
    # needs more than one slice-tile per CU (the 64 MiB hold exactly one 256x256 float32 tile per CU)
    M, N, K = 4352, 4352, 147456
    with torch.cuda.device(device):
        need = int(lib.mx_gemm_nt_workspace_bytes(M, N, K))
    assert need > 64 << 20
    # operands and output of the real size (zeros): were the call ever to launch, it would stay in
    # bounds and the status check below would be what fails
    codes = torch.zeros((M, K), dtype=torch.uint8, device=device)
    scales = torch.zeros(int(lib.mx_scales_mfma_bytes(M, K // 32)), dtype=torch.uint8, device=device)
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=device)
    for hook in (0, 3, 1):  # the size check does not depend on the kernel-selection hook
        lib.mx_debug_force_kernel(hook)
        with torch.cuda.device(device):
            st = lib.mx_gemm_nt_static(ops._ptr(codes), ops._ptr(scales), ops._ptr(codes), ops._ptr(scales),
                                       ops._ptr(out), M, N, K, N, ops._stream(out))
        lib.mx_debug_force_kernel(0)
        assert st == 5 and b"scratch" in lib.mx_status_string(st)
    torch.cuda.synchronize(device)
    assert bool((out == 7.0).all()), "nothing was launched"
