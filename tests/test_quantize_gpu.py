"""Parity of the fused rotate+quantize HIP kernels against the CPU oracle, through the C ABI.
Bar: packed E2M1 codes and scale bytes bit-exact (torch.equal)."""
import numpy as np
import pytest
import torch

from conftest import make_outlier_normal, make_student_t
from oracle import fpq_oracle as O

pytestmark = pytest.mark.gpu


def _check(x, fmt, rot="hadamard", g=128, zero=0, pad=False, gs=None, h=None):
    import capi
    kind = {"hadamard": O.ROT_HADAMARD, "identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR,
            "general": O.ROT_GENERAL}[rot]
    if fmt == "mxfp4":
        want_c, want_s, _ = O.quantize_mx(x, kind, g, h=h, zero_nibble=zero)
    else:
        want_c, want_s, _ = O.quantize_nv(x, gs, kind, g, h=h, zero_nibble=zero)
    got_c, got_s = capi.quantize(x, fmt, rot, g, global_scale=gs, zero_policy=zero, pad=pad, h=h)
    r, c = want_s.shape
    bad_c = (got_c != want_c).sum().item()
    bad_s = (got_s[:r, :c] != want_s).sum().item()
    assert bad_s == 0, f"{bad_s} scale bytes differ of {want_s.numel()}"
    assert bad_c == 0, f"{bad_c} code bytes differ of {want_c.numel()}"
    if pad:
        assert (got_s[r:, :] == 0).all() and (got_s[:, c:] == 0).all()


def test_device_e2m1_rounding_exhaustive():
    """Every bf16 bit pattern plus the fp32 neighbours of every decision point, both policies."""
    from fp_quant import _engine
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    v = bits.view(torch.bfloat16).float()
    v = v[~torch.isnan(v)]
    pts = []
    for m in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 0.5, 1.0, 2.0):
        b = int(np.float32(m).view(np.uint32))
        for d in range(-3, 4):
            f = np.uint32(b + d).view(np.float32)
            pts += [float(f), -float(f)]
    v = torch.cat([v, torch.tensor(pts, dtype=torch.float32)])
    vin = v.cuda()
    for policy in (O.ZERO_NIBBLE_REFERENCE, O.ZERO_NIBBLE_SIGNED):
        out = torch.empty(v.numel(), dtype=torch.uint8, device="cuda")
        st = _engine.lib().fpq_test_e2m1(vin.data_ptr(), out.data_ptr(), v.numel(), policy,
                                         torch.cuda.current_stream().cuda_stream)
        assert st == 0
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), O.e2m1_codes(v, policy))


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("zero", [0, 1])
def test_mx_small_all_block_sizes(g, zero):
    x = make_outlier_normal(96, 512, seed=100 + g)
    _check(x, "mxfp4", "hadamard", g, zero)


@pytest.mark.parametrize("g", [16, 32, 64, 128])
@pytest.mark.parametrize("zero", [0, 1])
def test_nv_small_all_block_sizes(g, zero):
    x = make_student_t(96, 512, seed=200 + g)
    gs = O.nv_tracked_global_scale(O.rotate(x, O.ROT_HADAMARD, g, float(O.hadamard_matrix(g)[0, 0])))
    _check(x, "nvfp4", "hadamard", g, zero, gs=gs)
    _check(x, "nvfp4", "hadamard", g, zero, gs=10.0)


def test_identity_rotation():
    x = make_outlier_normal(64, 256, seed=7)
    _check(x, "mxfp4", "identity", 32)
    _check(x, "nvfp4", "identity", 16, gs=10.0)


@pytest.mark.parametrize("rows,cols", [(1, 128), (3, 4096), (130, 384), (257, 128), (5, 32)])
def test_ragged_shapes_and_padding(rows, cols):
    x = make_outlier_normal(rows, cols, seed=rows * 7 + cols)
    g = 128 if cols % 128 == 0 else 32
    _check(x, "mxfp4", "hadamard", g, pad=True)
    _check(x, "mxfp4", "hadamard", 32, pad=False)
    _check(x, "nvfp4", "hadamard", 16, pad=True, gs=10.0)


@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_gsr_rotation(g):
    """Sequency-ordered Hadamard (transform_init="gsr"): small input (generic kernel) and an input
    large enough for the streaming kernel."""
    for rows in (40, (1 << 21) // 256 + 5):
        x = make_outlier_normal(rows, 256, seed=300 + g)
        if g >= 32:
            _check(x, "mxfp4", "gsr", g, zero=0)
        _check(x, "nvfp4", "gsr", g, zero=1, gs=3.0)


@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_general_rotation_matrix(g):
    """An arbitrary (non-symmetric) bf16 matrix: sequential fp32 fma accumulation, bit-exact."""
    gen = torch.Generator().manual_seed(400 + g)
    q, _ = torch.linalg.qr(torch.randn(g, g, generator=gen))
    h = q.to(torch.bfloat16)
    x = make_outlier_normal(48, 256, seed=500 + g)
    if g >= 32:
        _check(x, "mxfp4", "general", g, h=h)
    _check(x, "nvfp4", "general", g, gs=3.0, h=h, zero=1)


def test_empty_input():
    import capi
    x = torch.empty(0, 128, dtype=torch.bfloat16)
    c, s = capi.quantize(x, "mxfp4", "hadamard", 128)
    assert c.shape == (0, 64) and s.shape == (0, 4)


def test_adversarial_values():
    """Zero groups, powers of two, exact ties, tiny and huge magnitudes (slow scale path)."""
    gen = torch.Generator().manual_seed(9)
    rows = []
    base = torch.randn(128, generator=gen)
    rows.append(torch.zeros(128))                                   # all zero
    r = torch.zeros(128); r[5] = 1.0; rows.append(r)                # single spike
    rows.append(torch.full((128,), 2.0))                            # constant power of two
    r = base.clone(); r[:32] = 0; rows.append(r)                    # one zero group
    rows.append(base * 1e-30)                                       # tiny (a < 2^-98)
    rows.append(base * 1e-38)                                       # subnormal-range bf16
    rows.append(base * 1e30)                                        # large
    rows.append(base * 3e37)                                        # near bf16 max after rotation
    rows.append(torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 16))
    rows.append(-torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 16) * 8)
    r = torch.zeros(128); r[::2] = 1.0; r[1::2] = -1.0; rows.append(r)
    x = torch.stack(rows).to(torch.bfloat16)
    for zero in (0, 1):
        _check(x, "mxfp4", "identity", 32, zero)
        _check(x, "mxfp4", "hadamard", 32, zero)
        _check(x, "mxfp4", "hadamard", 128, zero)
        for gs in (10.0, 1.0, 2688.0 / 7.0, 1e-3, 1e4):
            _check(x[:7], "nvfp4", "identity", 16, zero, gs=gs)
            _check(x[:7], "nvfp4", "hadamard", 16, zero, gs=gs)
            _check(x[8:], "nvfp4", "identity", 16, zero, gs=gs)
            _check(x[8:], "nvfp4", "hadamard", 64, zero, gs=gs)


def _adversarial_rows(cols):
    gen = torch.Generator().manual_seed(19)
    base = torch.randn(cols, generator=gen)
    rows = [torch.zeros(cols), base * 1e-30, base * 1e-38, base * 1e30, base * 3e37, base,
            torch.full((cols,), 2.0), -torch.full((cols,), 0.0)]
    r = torch.zeros(cols); r[5] = 1.0; rows.append(r)
    r = base.clone(); r[: cols // 2] = 0; rows.append(r)
    r = torch.zeros(cols); r[::2] = 1.0; r[1::2] = -1.0; rows.append(r)
    rows.append(torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * (cols // 8)))
    rows.append(-torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * (cols // 8)) * 8)
    return torch.stack(rows)


@pytest.mark.parametrize("cols", [128, 192, 4096])
def test_streaming_kernel_adversarial_and_ragged(cols):
    """Inputs of >= 2^21 elements take the streaming kernel: adversarial rows (zero groups, tiny,
    huge, ties, negative zeros) scattered through random data, a row count that leaves a partial
    last tile, padded scale strides, every block size and both zero policies."""
    adv = _adversarial_rows(cols)
    n_rows = (1 << 21) // cols + 37
    x = make_outlier_normal(n_rows, cols, seed=cols).float()
    pos = torch.randperm(n_rows, generator=torch.Generator().manual_seed(3))[: adv.shape[0] * 3]
    for i, p in enumerate(pos.tolist()):
        x[p] = adv[i % adv.shape[0]]
    x[-1] = adv[2]
    x = x.to(torch.bfloat16)
    gs_mx = [g for g in (32, 64, 128) if cols % g == 0]
    for zero in (0, 1):
        for g in gs_mx:
            _check(x, "mxfp4", "hadamard", g, zero, pad=(g == 32))
        _check(x, "mxfp4", "identity", 32, zero)
        for g in [16] + gs_mx:
            _check(x, "nvfp4", "hadamard", g, zero, gs=10.0, pad=(g == 16))
        _check(x, "nvfp4", "identity", 16, zero, gs=3.0)
    _check(x, "nvfp4", "hadamard", 16, 0, gs=1e-25)   # global scale outside the fast range
    _check(x, "nvfp4", "hadamard", 16, 0, gs=1e-3)
    _check(x, "nvfp4", "hadamard", 16, 0, gs=2688.0 / 7.0)


def test_streaming_kernel_from_two_to_the_24_elements():
    """From 2^24 elements on a lane of the streaming kernel owns 64 elements instead of 32 (below, the test
    above): the same adversarial rows in a ragged input of that size."""
    cols = 4096
    adv = _adversarial_rows(cols)
    n_rows = (1 << 24) // cols + 37
    x = make_outlier_normal(n_rows, cols, seed=24).float()
    pos = torch.randperm(n_rows, generator=torch.Generator().manual_seed(5))[: adv.shape[0] * 3]
    for i, p in enumerate(pos.tolist()):
        x[p] = adv[i % adv.shape[0]]
    x[-1] = adv[2]
    x = x.to(torch.bfloat16)
    _check(x, "mxfp4", "hadamard", 128, 0)
    _check(x, "mxfp4", "hadamard", 32, 1, pad=True)
    _check(x, "mxfp4", "identity", 32, 0)
    _check(x, "nvfp4", "hadamard", 64, 0, gs=10.0)
    _check(x, "nvfp4", "identity", 16, 1, gs=3.0)
    _check(x, "nvfp4", "hadamard", 16, 0, gs=1e-25)   # global scale outside the fast range


def test_negative_zero_inputs_keep_their_sign_under_signed_policy():
    x = torch.zeros(64, 128)
    x[::2] = -0.0
    x[3, 5] = 1.0
    x[4, 7] = -1.0
    x = x.to(torch.bfloat16)
    for zero in (0, 1):
        _check(x, "mxfp4", "identity", 32, zero)
        _check(x, "nvfp4", "identity", 16, zero, gs=3.0)
        _check(x, "mxfp4", "hadamard", 32, zero)


def test_mx_tie_inputs_after_division():
    """Inputs whose scaled value lands exactly on, or one ulp beside, an E2M1 midpoint:
    x = t * fl(4/3) * 2^k is not bf16-representable in general, so use identity rotation on
    bf16 values with short mantissas and group maxima that put them on the decision points."""
    vals = []
    for k in (-3, 0, 5):
        for m in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0):
            grp = [0.0] * 32
            grp[0] = 4.0 * 2.0 ** k          # a = 2^(k+2) -> s = 2^k * fl(4/3)
            for j, t in enumerate((1.0, 1.0078125, 0.9921875)):
                grp[1 + j] = m * (4.0 / 3.0) * t * 2.0 ** k
                grp[4 + j] = -grp[1 + j]
            vals += grp
    x = torch.tensor(vals).view(-1, 32 * 3).to(torch.bfloat16)
    _check(x, "mxfp4", "identity", 32, 0)
    _check(x, "mxfp4", "identity", 32, 1)


def test_config1_mxfp4_full_size():
    x = make_outlier_normal(2048, 4096, seed=0)
    _check(x, "mxfp4", "hadamard", 128)


def test_config2_nvfp4_full_size():
    x = make_student_t(8192, 4096, seed=1)
    gs = O.nv_tracked_global_scale(O.rotate(x, O.ROT_HADAMARD, 16, 0.25))
    _check(x, "nvfp4", "hadamard", 16, gs=gs)


def test_rejects_bad_arguments():
    import capi
    x = torch.zeros(4, 96, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        capi.quantize(x, "mxfp4", "hadamard", 128)       # cols % g != 0
    with pytest.raises(ValueError):
        capi.quantize(x, "mxfp4", "hadamard", 48)        # unsupported block size
    with pytest.raises(ValueError):
        capi.quantize(x, "mxfp4", "hadamard", 32, zero_policy=7)
