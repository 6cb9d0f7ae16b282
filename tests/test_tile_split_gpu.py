"""K split inside the NVFP4 tile kernels (a few hundred rows on few weight rows: at most one 64 x 128 or
128 x 128 workgroup tile per CU).  With an even number of 256-K blocks the workgroup has eight waves in two
groups, each multiplying one half of K, and the halves meet in LDS (no workspace).  With an odd number and a
long K (fpq_gemm_nvf4_packed_splitk beyond 256 rows) K is cut across workgroups: fp32 parts of the workgroup
tiles meet in the caller's workspace and the workgroup that arrives last adds them in part order.  Checked: the
oracle's values (bias and residual included), the same bits on every repetition, counters left at zero, a
smaller workspace only means fewer parts, and the layer takes the same kernel eagerly, through the traced
operator and under a graph capture.
Reference contract: matmul_nvf4_bf16_tn_op (inference_lib/src/fp_quant/module/qutlass_ops.py:149-168)."""
import pytest
import torch

from fp_quant import _engine
from oracle import fpq_oracle as O
import capi
from conftest import needs_packed
from test_packed_gpu import pack_nv_by_definition

pytestmark = pytest.mark.gpu

ALPHA = 2.0 ** -6


def _operands(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(40, 64, (m, k // 16), dtype=torch.uint8, generator=g)
    ws = torch.randint(40, 64, (n, k // 16), dtype=torch.uint8, generator=g)
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=g) * 4).to(torch.bfloat16)
    return xq, xs, wq, ws, bias, res, g


# (rows, N, K), an odd number of 256-K blocks: 64 x 128 tiles in two and three parts, 128 x 128 tiles, ragged
# edges in both directions
SHAPES = [(300, 1024, 8448), (512, 4096, 12544), (384, 2048, 14592), (257, 200, 8448), (700, 520, 8448),
          (1000, 1024, 8448)]
# an even number of blocks: two groups of four waves per workgroup -- 64 x 128 and 128 x 128 tiles, one block per
# group up to 28, ragged edges, 129-256 rows on many weight rows
GROUP_SHAPES = [(512, 4096, 12288), (300, 4100, 8192), (1000, 1100, 2560), (384, 4096, 14336), (640, 4096, 4096),
                (200, 12288, 2048), (129, 16384, 2560), (513, 8190, 3072)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_tile_kernel_split_matches_the_oracle(m, n, k):
    lib = _engine.lib()
    need = int(lib.fpq_gemm_nvf4_packed_workspace_bytes(m, n, k))
    assert need > 16384, "the shape is expected to split K"
    xq, xs, wq, ws, bias, res, g = _operands(m, n, k, m + n + k)
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    workspace = torch.zeros(need, dtype=torch.uint8, device="cuda")
    y = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res, workspace=workspace, nv=True)
    assert not workspace[:16384].any()
    ri = torch.cat([torch.tensor([0, 127, 128, m - 1]), torch.randperm(m, generator=g)[:40]]).unique()
    ci = torch.cat([torch.tensor([0, 63, 64, 127, 128, n - 1]), torch.randperm(n, generator=g)[:160]]).unique()
    ref, mag = O.gemm_ref(xq[ri], xs[ri], wq[ci], ws[ci], ALPHA, "nvfp4")
    want = (ref.to(torch.bfloat16) + bias[ci]) + res[ri][:, ci]
    got = y[ri][:, ci]
    tol = 2.0 ** -7 * torch.maximum(want.double().abs(), ref.abs()) + 2.0 ** -7 * res[ri][:, ci].double().abs() + 1e-5 * mag + 1e-6
    assert ((got.double() - want.double()).abs() <= tol).all()
    assert (got.view(torch.int16) == want.view(torch.int16)).double().mean() > 0.95
    # deterministic: the parts are added in part order whatever the order of arrival
    for _ in range(3):
        again = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res, workspace=workspace,
                                        nv=True)
        assert torch.equal(again.view(torch.int16), y.view(torch.int16))
    assert not workspace[:16384].any()
    # K whole (no workspace): the same values within the tolerance, summed in another order
    whole = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res)
    assert ((whole[ri][:, ci].double() - want.double()).abs() <= tol).all()
    # a workspace too small for every part: fewer parts (or none), never an error, the same tolerance
    small = torch.zeros(16384 + (need - 16384) // 2 // 256 * 256, dtype=torch.uint8, device="cuda")
    fewer = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res, workspace=small, nv=True)
    assert ((fewer[ri][:, ci].double() - want.double()).abs() <= tol).all() and not small[:16384].any()


@pytest.mark.parametrize("m,n,k", GROUP_SHAPES)
def test_two_groups_per_workgroup_match_the_oracle(m, n, k):
    lib = _engine.lib()
    xq, xs, wq, ws, bias, res, g = _operands(m, n, k, m + n + k)
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    y = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res)
    ri = torch.cat([torch.tensor([0, 127, 128, m - 1]), torch.randperm(m, generator=g)[:40]]).unique()
    ci = torch.cat([torch.tensor([0, 63, 64, 127, 128, n - 1]), torch.randperm(n, generator=g)[:160]]).unique()
    ref, mag = O.gemm_ref(xq[ri], xs[ri], wq[ci], ws[ci], ALPHA, "nvfp4")
    want = (ref.to(torch.bfloat16) + bias[ci]) + res[ri][:, ci]
    got = y[ri][:, ci]
    tol = 2.0 ** -7 * torch.maximum(want.double().abs(), ref.abs()) + 2.0 ** -7 * res[ri][:, ci].double().abs() + 1e-5 * mag + 1e-6
    assert ((got.double() - want.double()).abs() <= tol).all()
    assert (got.view(torch.int16) == want.view(torch.int16)).double().mean() > 0.95
    for _ in range(3):   # the halves are added in a fixed order
        again = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res)
        assert torch.equal(again.view(torch.int16), y.view(torch.int16))
    # a workspace changes nothing: these shapes need none
    if m > 256:
        assert int(lib.fpq_gemm_nvf4_packed_workspace_bytes(m, n, k)) == 0
    workspace = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    same = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias, residual=res, workspace=workspace, nv=True)
    if m > 256:
        assert torch.equal(same.view(torch.int16), y.view(torch.int16)) and not workspace.any()
    # without bias and residual as well
    plain = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, ALPHA)
    want0 = ref.to(torch.bfloat16)
    assert ((plain[ri][:, ci].double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6).all()
    assert (plain[ri][:, ci] == want0).double().mean() > 0.97


def test_workspace_size_function():
    lib = _engine.lib()
    size = lib.fpq_gemm_nvf4_packed_workspace_bytes
    assert size(512, 4096, 12544) == 16384 + 2 * 256 * 32768       # 4 x 64 tiles of 64 x 128, 49 blocks of K in two parts
    assert size(512, 4096, 12288) == 0                             # 48 blocks: halved inside the workgroups
    assert size(512, 4096, 4096) == 0                              # K too short to cut across workgroups
    assert size(4096, 4096, 12288) == 0                            # enough tiles without
    assert size(64, 4096, 12288) == lib.fpq_gemm_mxf4_packed_workspace_bytes(64, 4096, 12288) > 0
    assert size(200, 4096, 12288) == lib.fpq_gemm_mxf4_packed_workspace_bytes(128, 4096, 12288)   # two passes of 128 / 72 rows
    assert lib.fpq_gemm_mxf4_packed_workspace_bytes(512, 4096, 14336) == 0   # MXFP4 never splits in the tile kernels


@needs_packed
def test_layer_takes_the_split_on_every_call_path():
    """An NVFP4 FPQuantLinear with few output features and a long K at 300 rows: eager call (the stream's own
    workspace), the traced operator and a graph capture on a side stream (the layer's workspace) give the same
    bits, which are those of the C entry point with a workspace of its own."""
    import fp_quant
    from fp_quant.module import eager
    k, n, m = 8448, 512, 300
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.NVFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=16)
    torch.manual_seed(3)
    lin = fp_quant.FPQuantLinear(k, n, cfg, bias=True, device="cuda", dtype=torch.bfloat16)
    lin.weight.data.normal_(0, 0.02)
    lin.bias.data.normal_()
    lin.pre_forward()
    own = getattr(lin.qweight, "_fpq_splitk", None)
    need = int(_engine.lib().fpq_gemm_nvf4_packed_workspace_bytes(m, n, k))
    assert need > 16384 and own is not None and own.numel() >= need
    x = torch.randn(m, k, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        y = lin(x)
        op = eager.linear_w4a4_op(x, lin.forward_hadamard_matrix, lin.qweight, lin.scales, lin.weight_global_scale,
                                  lin.act_global_scale, lin.bias, True)
        assert torch.equal(op, y)
        graph = torch.cuda.CUDAGraph()
        static_x = x.clone()
        with torch.cuda.graph(graph):
            static_y = lin(static_x)
        for _ in range(2):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, y)
    assert not own[:16384].any()
    sd = lin.state_dict()
    xq, xs = capi.quantize(x.cpu(), "nvfp4", "hadamard", 16, global_scale=float(lin.act_global_scale))
    xp, xsp = capi.pack_nv(xq, xs)
    wp, wsp = capi.pack_nv(sd["qweight"].cpu(), sd["scales"].cpu())
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    workspace = torch.zeros(need, dtype=torch.uint8, device="cuda")
    direct = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=lin.bias.detach().cpu(), workspace=workspace,
                                     nv=True)
    assert torch.equal(direct, y.cpu())
    # K whole sums in another order: equal up to the rounding of a few fp32 sums (products of FP4 codes and E4M3
    # scales are exact and most partial sums too, so the bits often agree altogether)
    whole = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=lin.bias.detach().cpu())
    assert ((whole.double() - direct.double()).abs() <= 2.0 ** -7 * direct.double().abs() + 1e-3).all()
