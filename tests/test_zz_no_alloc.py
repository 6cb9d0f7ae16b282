"""fpq_gemm_mxf4_packed_noalloc (split-K counters and partial tiles in the library's own file-scope
device array) against fpq_gemm_mxf4_packed_splitk with a caller workspace: bit-equal outputs on calls
in a row that share the array, the later ones with smaller inputs; against the oracle on a shape that
splits; recorded into a HIP graph after fpq_prepare_device; counters back at zero after every call."""
import pytest
import torch

from fp_quant import _engine
from oracle import fpq_oracle as O
import capi
from test_packed_gpu import pack_by_definition

pytestmark = pytest.mark.gpu

ALPHA = 0.111328125


def _case(m, n, k, seed, row_major=False):
    g = torch.Generator().manual_seed(seed)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
    if row_major:
        return [t.cuda() for t in (xp, xsp, wp, wsp)], bias.cuda(), res.cuda(), (xq, xs, wq, ws)
    return [t.cuda() for t in (xp, xsp, wp, wsp)], bias.cuda(), res.cuda()


def _counters_are_zero():
    out = torch.full((16384,), 0xCD, dtype=torch.uint8, device="cuda")
    st = _engine.lib().fpq_test_noalloc_counters(out.data_ptr(), out.numel(), torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_test_noalloc_counters")
    torch.cuda.synchronize()
    return not bool(out.any())


def _noalloc(ops, m, n, k, bias, res):
    lib = _engine.lib()
    alpha = torch.tensor([ALPHA], dtype=torch.float32, device="cuda")
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    st = lib.fpq_gemm_mxf4_packed_noalloc(*(t.data_ptr() for t in ops), alpha.data_ptr(),
                                          bias.data_ptr() if bias is not None else None,
                                          res.data_ptr() if res is not None else None, y.data_ptr(), m, n, k,
                                          torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_gemm_mxf4_packed_noalloc")
    return y


def _with_workspace(ops, m, n, k, bias, res):
    need = _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes(m, n, k)
    wspace = torch.zeros(max(need, 256), dtype=torch.uint8, device="cuda")
    return capi.gemm_packed_splitk(*ops, m, n, k, ALPHA, bias=bias, residual=res, workspace=wspace).cuda()


# K split in two and in three, the largest split the array holds (four activation row tiles, 4 MB of partial
# tiles), then smaller inputs on the same array: a split over fewer weight tiles,
# K whole (no scratch use), two activation row tiles, and the 128x128 tile kernel
SEQUENCE = [(16, 4096, 14336), (8, 1024, 14336), (128, 4096, 8192), (5, 257, 12288), (1, 32, 8192), (32, 2048, 4096),
            (64, 8200, 512), (128, 8320, 256), (17, 515, 9216), (64, 515, 9216)]


def test_noalloc_equals_workspace_entry_on_calls_in_a_row():
    need = _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes
    assert need(*SEQUENCE[0]) > 16384 and need(*SEQUENCE[1]) > 16384     # both really split K
    cases = [(_case(m, n, k, 90 + i), (m, n, k)) for i, (m, n, k) in enumerate(SEQUENCE)]
    got = []
    for (ops, bias, res), (m, n, k) in cases:            # back to back on one stream, nothing in between
        got.append(_noalloc(ops, m, n, k, None, None))
        got.append(_noalloc(ops, m, n, k, bias, res))
    assert _counters_are_zero()
    it = iter(got)
    for (ops, bias, res), (m, n, k) in cases:
        y, yr = next(it), next(it)
        assert not torch.isnan(y.float()).any()
        assert torch.equal(y.view(torch.int16), _with_workspace(ops, m, n, k, None, None).view(torch.int16)), (m, n, k)
        assert torch.equal(yr.view(torch.int16), _with_workspace(ops, m, n, k, bias, res).view(torch.int16)), (m, n, k)


def test_noalloc_repeats_bit_identically():
    (ops, bias, res), (m, n, k) = _case(16, 4096, 14336, 7), (16, 4096, 14336)
    first = _noalloc(ops, m, n, k, bias, None)
    for _ in range(5):
        assert torch.equal(_noalloc(ops, m, n, k, bias, None).view(torch.int16), first.view(torch.int16))


@pytest.mark.parametrize("m,n,k", [(16, 4096, 14336), (100, 1024, 8192)])
def test_noalloc_matches_the_oracle_on_shapes_that_split(m, n, k):
    """Not only equal to the workspace entry point (which runs the same kernel and plan): the values are the
    oracle's, with bias and residual, on shapes whose K is split across workgroups."""
    assert _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes(m, n, k) > 16384
    ops, bias, res, (xq, xs, wq, ws) = _case(m, n, k, 300 + m, row_major=True)
    y = _noalloc(ops, m, n, k, bias, res).cpu()
    assert _counters_are_zero()
    gen = torch.Generator().manual_seed(m)
    ci = torch.cat([torch.tensor([0, 31, 32, n - 33, n - 32, n - 1]), torch.randperm(n, generator=gen)[:250]]).unique()
    ref, mag = O.gemm_ref(xq, xs, wq[ci], ws[ci], ALPHA, "mxfp4")
    want = (ref.to(torch.bfloat16) + bias.cpu()[ci]) + res.cpu()[:, ci]          # two separate bf16 additions
    assert torch.equal(y[:, ci].view(torch.int16), want.view(torch.int16)) or \
        ((y[:, ci].double() - want.double()).abs() <= 2.0 ** -7 * torch.maximum(want.double().abs(), ref.abs())
         + 1e-5 * mag + 1e-6).all()
    assert (y[:, ci].view(torch.int16) == want.view(torch.int16)).double().mean() > 0.97


def test_noalloc_recorded_into_a_graph_after_prepare_device():
    """The use the entry point is for: fpq_prepare_device outside the capture (it looks the scratch address
    up), then the call recorded into a HIP graph (it allocates nothing and records no memset); every replay,
    with eager work of the same entry point in between, gives the eager bits and leaves the counters at zero."""
    lib = _engine.lib()
    m, n, k = 8, 1024, 14336
    assert lib.fpq_gemm_mxf4_packed_workspace_bytes(m, n, k) > 16384
    ops, bias, res = _case(m, n, k, 77)
    other_ops, other_bias, _ = _case(16, 4096, 14336, 78)
    side = torch.cuda.Stream()
    assert lib.fpq_prepare_device(side.cuda_stream) == 0
    alpha = torch.tensor([ALPHA], dtype=torch.float32, device="cuda")
    want = _noalloc(ops, m, n, k, bias, None)
    torch.cuda.synchronize()
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = lib.fpq_gemm_mxf4_packed_noalloc(*(t.data_ptr() for t in ops), alpha.data_ptr(), bias.data_ptr(), None,
                                              y.data_ptr(), m, n, k, torch.cuda.current_stream().cuda_stream)
        assert st == 0
    for _ in range(4):
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), want.view(torch.int16))
        assert _counters_are_zero()
        _noalloc(other_ops, 16, 4096, 14336, other_bias, None)      # eager use of the same array in between
        torch.cuda.synchronize()


def test_noalloc_rejects_sizes_beyond_its_maximum():
    lib = _engine.lib()
    assert lib.fpq_gemm_mxf4_packed_noalloc_max_rows() == 128
    (ops, bias, res) = _case(129, 64, 256, 3)
    with pytest.raises(ValueError, match="beyond the stated maximum"):
        _noalloc(ops, 129, 64, 256, None, None)
    with pytest.raises(ValueError):                       # the argument checks of the workspace entry point
        _noalloc(ops, 128, 64, 200, None, None)
