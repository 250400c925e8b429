"""mi355_quant_dot_static: the quant_dot entry point that allocates nothing.  Its split-K partial
sums go to the library's static device buffer instead of a caller's workspace; the result must
be the bits mi355_quant_dot_ws gives with a workspace of the caller's (same kernels, same share
count), call after call, also when a smaller problem follows a larger one in the same buffer."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _operands(m, n, k, trans_b, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, generator=g).cuda()
    b = torch.randint(-128, 128, (n, k) if trans_b else (k, n), dtype=torch.int8, generator=g).cuda()
    return a, (b.t() if trans_b else b)


def test_two_calls_in_a_row_second_one_smaller(ops):
    # (128, 8192, 8192) fills the static buffer to its last byte; (16, 1024, 4096) then reuses
    # its first quarter MiB with the larger call's partial sums still in it
    for m, n, k, trans_b in ((128, 8192, 8192, False), (16, 1024, 4096, True)):
        print("static scratch", m, n, k, trans_b, flush=True)
        a, b = _operands(m, n, k, trans_b, m + n)
        need = ops.quant_dot_workspace_size(m, n, k, 1, trans_b)
        assert 0 < need <= STATIC_BYTES
        ws = torch.full((need,), 0x33, dtype=torch.uint8, device="cuda")
        want = ops.quant_dot(a, b, workspace=ws)
        got = torch.empty_like(want)
        # the first call on a device looks the buffer up (its code object is loaded then, which is
        # when the device gets its copy of the buffer); no later call changes the free memory
        ops.quant_dot(a, b, workspace="static", out=got)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        got.fill_(-1)
        ops.quant_dot(a, b, workspace="static", out=got)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before      # nothing was allocated or freed
        assert torch.equal(got, want)
        rows = [0, m // 2, m - 1]
        bm = b.cpu().numpy()
        assert np.array_equal(got[rows].cpu().numpy(), orc.quant_dot(a[rows].cpu().numpy(), bm, orc.I8))
        # the fused linear layer through the same buffer: per-column scales, zero points, bias, bf16
        sa = torch.full((1,), 0.02, device="cuda")
        sb = torch.rand(n, device="cuda") * 0.01 + 0.001
        bias = torch.randn(n, device="cuda")
        kw = dict(scale_a=sa, scale_b=sb, bias=bias, out_dtype=torch.bfloat16)
        want16 = ops.quant_dot(a, b, workspace=ws, **kw)
        got16 = ops.quant_dot(a, b, workspace="static", **kw)
        assert torch.equal(got16.view(torch.int16), want16.view(torch.int16))


def test_fp8_split_through_the_static_buffer(ops):
    for m, n, k in ((128, 768, 3072), (16, 512, 2048)):
        g = torch.Generator().manual_seed(k)
        a = (torch.randint(0, 256, (m, k), dtype=torch.uint8, generator=g) & 0x77).cuda()
        b = (torch.randint(0, 256, (k, n), dtype=torch.uint8, generator=g) & 0x77).cuda()
        need = ops.quant_dot_workspace_size(m, n, k, fp8=True)
        assert 0 < need <= STATIC_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = ops.quant_dot(a, b, fp8=True, workspace=ws)
        got = ops.quant_dot(a, b, fp8=True, workspace="static")
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))


def test_shapes_without_a_split_and_shapes_beyond_the_buffer(ops):
    from amdmigraphx_amd import Mi355Error
    # no split: the one-pass kernel, no scratch memory involved
    a, b = _operands(512, 512, 512, False, 3)
    assert ops.quant_dot_workspace_size(512, 512, 512) == 0
    assert torch.equal(ops.quant_dot(a, b, workspace="static"), ops.quant_dot(a, b))
    # a split that needs more than the buffer holds is refused, and nothing is written
    m, n, k = 255, 8192, 8192
    assert ops.quant_dot_workspace_size(m, n, k) > STATIC_BYTES
    a, b = _operands(m, n, k, False, 4)
    out = torch.full((m, n), -7, dtype=torch.int32, device="cuda")
    with pytest.raises(Mi355Error, match="static buffer"):
        ops.quant_dot(a, b, workspace="static", out=out)
    torch.cuda.synchronize()
    assert (out == -7).all()
